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
//     (scalar loads / SGPR operands).
//
//   A-type applications (1 -> SC channels: A(x), A(t1), A(gt1)) are gathered from the
//   rings; K-type applications (SC -> 1 channel: K(s), K(gn), K(gd)) are scattered plane by
//   plane into per-thread accumulators of the KD pending output planes, so each staged
//   value is read from LDS once per (row, tap-column) and reused for all tap planes.
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

// =================================================================== forward

template <int KD_, int KH_, int KW_, int SC_, int RH_, typename T> struct FwdKernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int RHK = RH + (PH > 0 ? 1 : 0);   // rows of t1 a thread produces
    static constexpr int NZR = RH + (PH > 0 ? 2 : 0);   // rows of s a thread stages
    static constexpr int NXR = RH + (PH > 0 ? 1 : 0);   // rows of x a thread stages
    static constexpr int XR = KD + 1;                   // x ring slots
    typedef FwdParams<T> Params;

    struct State {
        int strip, col, active;
        float t1acc[KD][RHK];
        float sdel[KD][RH][SC];
        float pz[SC][NZR];
        float px[NXR];
    };

    static NDC_HD int rows_s(int S) { return S * RHK + 2 * PH; }
    static NDC_HD int rows_x(int S) { return S * RH + 2 * PH; }
    static NDC_HD int rows_t(int S) { return S * RHK; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        return (SC * rows_s(t.S) + XR * rows_x(t.S) + KD * rows_t(t.S)) * t.P;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RS = rows_s(S), RX = rows_x(S), RT = rows_t(S);
        const int off_s = 0, off_x = SC * RS * P, off_t = off_x + XR * RX * P;
        const int total = off_t + KD * RT * P;
        const long long plane = (long long)H * W;
        const long long xbase = ((long long)id.b * p.C + id.c) * D * plane;
        const long long zbase = ((long long)id.b * p.C + id.c) * SC * D * plane;
        const float *hw = p.h + (long long)id.c * SC * KT;
        const float *bias = p.bias ? p.bias + id.c * SC : nullptr;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;

        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            const bool zin = k < D;
#pragma unroll
            for (int i = 0; i < SC; ++i) {
                const float bv = bias ? bias[i] : 0.f;
#pragma unroll
                for (int n = 0; n < NZR; ++n) {
                    const int j = st.strip + n * S, row = r0 - 2 * PH + j;
                    float v = 0.f;
                    if (zin && j < TH + 4 * PH && row >= 0 && row < H) {
                        v = Elem<T>::load(p.z + zbase + ((long long)i * D + k) * plane +
                                          (long long)row * W + st.col) + bv;
                        if (p.relu) v = v > 0.f ? v : 0.f;
                    }
                    st.pz[i][n] = v;
                }
            }
            const int kx = k - PD;
            const bool xin = kx >= 0 && kx < D;
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S, row = r0 - PH + j;
                float v = 0.f;
                if (xin && j < TH + 2 * PH && row >= 0 && row < H)
                    v = Elem<T>::load(p.x + xbase + (long long)kx * plane + (long long)row * W + st.col);
                st.px[n] = v;
            }
        };

        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
#pragma unroll
            for (int i = 0; i < SC; ++i)
#pragma unroll
                for (int n = 0; n < NZR; ++n) {
                    const int j = st.strip + n * S;
                    if (j < TH + 4 * PH) ex.st_(off_s + (i * RS + j) * P + PW + st.col, st.pz[i][n]);
                }
            const int slot = wrap((k - PD) % XR, XR);
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < TH + 2 * PH) ex.st_(off_x + (slot * RX + j) * P + PW + st.col, st.px[n]);
            }
        };

        // ---- set-up: thread coordinates, zeroed state, zeroed LDS (halo columns stay zero)
        ex.each([&](State &st, int tid) {
            st.strip = tid / W;
            st.col = tid - st.strip * W;
            st.active = st.strip < S;
#pragma unroll
            for (int a = 0; a < KD; ++a) {
#pragma unroll
                for (int r = 0; r < RHK; ++r) st.t1acc[a][r] = 0.f;
#pragma unroll
                for (int r = 0; r < RH; ++r)
#pragma unroll
                    for (int i = 0; i < SC; ++i) st.sdel[a][r][i] = 0.f;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + 2 * PD; ++k) {
            ex.each([&](State &st, int) {
                store_plane(st, k);
                load_plane(st, k + 1);
            });
            ex.sync();

            // ---- K-scatter: plane k of s feeds the KD pending planes of t1
            ex.each([&](State &st, int) {
                if (!st.active) return;
                if (k < D) {
#pragma unroll
                    for (int i = 0; i < SC; ++i)
#pragma unroll
                        for (int q = 0; q < RHK + 2 * PH; ++q)
#pragma unroll
                            for (int tw = 0; tw < KW; ++tw) {
                                const float v = ex.ld(off_s + (i * RS + st.strip * RHK + q) * P + st.col + tw);
#pragma unroll
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - th;
                                    if (rr < 0 || rr >= RHK) continue;
#pragma unroll
                                    for (int jd = 0; jd < KD; ++jd)
                                        st.t1acc[jd][rr] +=
                                            v * hw[((i * KD + (KD - 1 - jd)) * KH + th) * KW + tw];
                                }
                            }
#pragma unroll
                    for (int r = 0; r < RH; ++r)
#pragma unroll
                        for (int i = 0; i < SC; ++i)
                            st.sdel[KD - 1][r][i] =
                                ex.ld(off_s + (i * RS + st.strip * RH + r + 2 * PH) * P + PW + st.col);
                } else {
#pragma unroll
                    for (int r = 0; r < RH; ++r)
#pragma unroll
                        for (int i = 0; i < SC; ++i) st.sdel[KD - 1][r][i] = 0.f;
                }
                // plane k - PD of t1 is complete: publish it (zero outside the volume)
                const int pf = k - PD;
                const bool inplane = pf >= 0 && pf < D;
                const int slot = wrap(pf % KD, KD);
#pragma unroll
                for (int r = 0; r < RHK; ++r) {
                    const int j = st.strip * RHK + r, row = r0 - PH + j;
                    const bool live = inplane && row >= 0 && row < H;
                    const float v = live ? st.t1acc[0][r] : 0.f;
                    ex.st_(off_t + (slot * RT + j) * P + PW + st.col, v);
                    if (p.t1 && live && j >= PH && j < PH + TH)
                        Elem<T>::store(p.t1 + xbase + (long long)pf * plane + (long long)row * W + st.col, v);
#pragma unroll
                    for (int a = 0; a + 1 < KD; ++a) st.t1acc[a][r] = st.t1acc[a + 1][r];
                    st.t1acc[KD - 1][r] = 0.f;
                }
            });
            ex.sync();

            // ---- A-gather + epilogue for output plane k - 2*PD
            ex.each([&](State &st, int) {
                if (!st.active) return;
                const int j0 = k - 2 * PD;
                if (j0 >= 0) {
                    float an[SC][RH], ad[SC][RH];
#pragma unroll
                    for (int i = 0; i < SC; ++i)
#pragma unroll
                        for (int r = 0; r < RH; ++r) an[i][r] = ad[i][r] = 0.f;
#pragma unroll
                    for (int td = 0; td < KD; ++td) {
                        const int pl = j0 + PD - td;
                        const int bx = off_x + wrap(pl % XR, XR) * RX * P;
                        const int bt = off_t + wrap(pl % KD, KD) * RT * P;
#pragma unroll
                        for (int q = 0; q < RH + 2 * PH; ++q)
#pragma unroll
                            for (int tw = 0; tw < KW; ++tw) {
                                const int o = (st.strip * RH + q) * P + st.col + 2 * PW - tw;
                                const float vx = ex.ld(bx + o), vt = ex.ld(bt + o);
#pragma unroll
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - 2 * PH + th;
                                    if (rr < 0 || rr >= RH) continue;
#pragma unroll
                                    for (int i = 0; i < SC; ++i) {
                                        const float wv = hw[((i * KD + td) * KH + th) * KW + tw];
                                        an[i][rr] += vx * wv;
                                        ad[i][rr] += vt * wv;
                                    }
                                }
                            }
                    }
#pragma unroll
                    for (int r = 0; r < RH; ++r) {
                        const int row = r0 + st.strip * RH + r;
                        if (row >= H) continue;
#pragma unroll
                        for (int i = 0; i < SC; ++i) {
                            const float v = st.sdel[0][r][i] * (an[i][r] + p.eps) * fast_rcp(ad[i][r] + p.eps);
                            Elem<T>::store(p.out + zbase + ((long long)i * D + j0) * plane +
                                               (long long)row * W + st.col, v);
                        }
                    }
                }
#pragma unroll
                for (int a = 0; a + 1 < KD; ++a)
#pragma unroll
                    for (int r = 0; r < RH; ++r)
#pragma unroll
                        for (int i = 0; i < SC; ++i) st.sdel[a][r][i] = st.sdel[a + 1][r][i];
            });
        }
    }
};

// =================================================================== backward, pass 1

template <int KD_, int KH_, int KW_, int SC_, int RH_, typename T> struct Bwd1Kernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int RHG = RH + (PH > 0 ? 1 : 0);   // rows of gn/gd a thread produces
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

    static NDC_HD int rows_x(int S) { return S * RHG + 2 * PH; }
    static NDC_HD int rows_g(int S) { return S * RHG; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = (2 * XR * rows_x(t.S) + 2 * SC * rows_g(t.S)) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(S), RG = rows_g(S);
        const int off_x = 0, off_t = XR * RX * P, off_g = 2 * XR * RX * P;
        const int total = off_g + 2 * SC * RG * P;
        const long long plane = (long long)H * W;
        const long long xbase = ((long long)id.b * p.C + id.c) * D * plane;
        const long long zbase = ((long long)id.b * p.C + id.c) * SC * D * plane;
        const float *hw = p.h + (long long)id.c * SC * KT;
        const float *bias = p.bias ? p.bias + id.c * SC : nullptr;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;

        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            const bool in = k >= 0 && k < D;
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S, row = r0 - 2 * PH + j;
                float vx = 0.f, vt = 0.f;
                if (in && j < TH + 4 * PH && row >= 0 && row < H) {
                    const long long o = xbase + (long long)k * plane + (long long)row * W + st.col;
                    vx = Elem<T>::load(p.x + o);
                    vt = Elem<T>::load(p.t1 + o);
                }
                st.px[n] = vx;
                st.pt[n] = vt;
            }
        };
        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
            const int slot = wrap(k % XR, XR);
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < TH + 4 * PH) {
                    ex.st_(off_x + (slot * RX + j) * P + PW + st.col, st.px[n]);
                    ex.st_(off_t + (slot * RX + j) * P + PW + st.col, st.pt[n]);
                }
            }
        };

        ex.each([&](State &st, int tid) {
            st.strip = tid / W;
            st.col = tid - st.strip * W;
            st.active = st.strip < S;
#pragma unroll
            for (int i = 0; i < SC; ++i)
#pragma unroll
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
#pragma unroll
            for (int a = 0; a < KD; ++a)
#pragma unroll
                for (int r = 0; r < RH; ++r) st.accx[a][r] = st.acct[a][r] = 0.f;
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + 2 * PD; ++k) {
            ex.each([&](State &st, int) {
                store_plane(st, k);
                load_plane(st, k + 1);
            });
            ex.sync();

            // ---- gather: n, d, gn, gd of plane k - PD on the band + one halo row each side
            const int j1 = k - PD;
            const bool live1 = j1 >= 0 && j1 < D;
            ex.each([&](State &st, int) {
                if (!st.active || !live1) return;
                // own-position operands come straight from global memory
                float sv[SC][RHG], gv[SC][RHG];
#pragma unroll
                for (int r = 0; r < RHG; ++r) {
                    const int j = st.strip * RHG + r, row = r0 - PH + j;
                    const bool in = j < TH + 2 * PH && row >= 0 && row < H;
#pragma unroll
                    for (int i = 0; i < SC; ++i) {
                        float s = 0.f, g = 0.f;
                        if (in) {
                            const long long o = zbase + ((long long)i * D + j1) * plane +
                                                (long long)row * W + st.col;
                            s = Elem<T>::load(p.z + o) + (bias ? bias[i] : 0.f);
                            if (p.relu) s = s > 0.f ? s : 0.f;
                            g = Elem<T>::load(p.gout + o);
                        }
                        sv[i][r] = s;
                        gv[i][r] = g;
                    }
                }
                float an[SC][RHG], ad[SC][RHG];
#pragma unroll
                for (int i = 0; i < SC; ++i)
#pragma unroll
                    for (int r = 0; r < RHG; ++r) an[i][r] = ad[i][r] = 0.f;
#pragma unroll
                for (int td = 0; td < KD; ++td) {
                    const int slot = wrap((j1 + PD - td) % XR, XR);
#pragma unroll
                    for (int q = 0; q < RHG + 2 * PH; ++q)
#pragma unroll
                        for (int tw = 0; tw < KW; ++tw) {
                            const int o = (slot * RX + st.strip * RHG + q) * P + st.col + 2 * PW - tw;
                            const float vx = ex.ld(off_x + o), vt = ex.ld(off_t + o);
#pragma unroll
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 * PH + th;
                                if (rr < 0 || rr >= RHG) continue;
#pragma unroll
                                for (int i = 0; i < SC; ++i) {
                                    const float wv = hw[((i * KD + td) * KH + th) * KW + tw];
                                    an[i][rr] += vx * wv;
                                    ad[i][rr] += vt * wv;
                                }
                            }
                        }
                }
                // gn, gd; publish them for the scatter; keep own-band copies for the filter gradient
#pragma unroll
                for (int r = 0; r < RHG; ++r) {
                    const int j = st.strip * RHG + r;
                    const bool own = j >= PH && j < PH + TH;
#pragma unroll
                    for (int i = 0; i < SC; ++i) {
                        const float inv = fast_rcp(ad[i][r] + p.eps);
                        const float gn = gv[i][r] * sv[i][r] * inv;
                        const float gd = -(gn * (an[i][r] + p.eps)) * inv;
                        ex.st_(off_g + (i * RG + j) * P + PW + st.col, gn);
                        ex.st_(off_g + ((SC + i) * RG + j) * P + PW + st.col, gd);
                        an[i][r] = own ? gn : 0.f;
                        ad[i][r] = own ? gd : 0.f;
                    }
                }
                if (p.need_gh) {
#pragma unroll
                    for (int td = 0; td < KD; ++td) {
                        const int slot = wrap((j1 + PD - td) % XR, XR);
#pragma unroll
                        for (int q = 0; q < RHG + 2 * PH; ++q)
#pragma unroll
                            for (int tw = 0; tw < KW; ++tw) {
                                const int o = (slot * RX + st.strip * RHG + q) * P + st.col + 2 * PW - tw;
                                const float vx = ex.ld(off_x + o), vt = ex.ld(off_t + o);
#pragma unroll
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - 2 * PH + th;
                                    if (rr < 0 || rr >= RHG) continue;
#pragma unroll
                                    for (int i = 0; i < SC; ++i)
                                        st.gacc[i][(td * KH + th) * KW + tw] +=
                                            an[i][rr] * vx + ad[i][rr] * vt;
                                }
                            }
                    }
                }
            });
            ex.sync();

            // ---- scatter: plane k - PD of gn/gd feeds the pending planes of gx / gt1
            ex.each([&](State &st, int) {
                if (!st.active) return;
                if (live1) {
#pragma unroll
                    for (int i = 0; i < SC; ++i)
#pragma unroll
                        for (int q = 0; q < RH + 2 * PH; ++q)
#pragma unroll
                            for (int tw = 0; tw < KW; ++tw) {
                                const int o = (st.strip * RH + q) * P + st.col + tw;
                                const float vn = ex.ld(off_g + i * RG * P + o);
                                const float vd = ex.ld(off_g + (SC + i) * RG * P + o);
#pragma unroll
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - th;
                                    if (rr < 0 || rr >= RH) continue;
#pragma unroll
                                    for (int jd = 0; jd < KD; ++jd) {
                                        const float wv = hw[((i * KD + (KD - 1 - jd)) * KH + th) * KW + tw];
                                        st.accx[jd][rr] += vn * wv;
                                        st.acct[jd][rr] += vd * wv;
                                    }
                                }
                            }
                }
                const int pf = k - 2 * PD;
#pragma unroll
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    if (pf >= 0 && row < H) {
                        const long long o = xbase + (long long)pf * plane + (long long)row * W + st.col;
                        if (p.gx) Elem<T>::store(p.gx + o, st.accx[0][r]);
                        Elem<T>::store(p.gt1 + o, st.acct[0][r]);
                    }
#pragma unroll
                    for (int a = 0; a + 1 < KD; ++a) {
                        st.accx[a][r] = st.accx[a + 1][r];
                        st.acct[a][r] = st.acct[a + 1][r];
                    }
                    st.accx[KD - 1][r] = 0.f;
                    st.acct[KD - 1][r] = 0.f;
                }
            });
        }

        if (p.need_gh) {
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

    static NDC_HD int rows_x(int S) { return S * RH + 2 * PH; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = 3 * XR * rows_x(t.S) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(S);
        const int off_x = 0, off_t = XR * RX * P, off_g = 2 * XR * RX * P;
        const int total = 3 * XR * RX * P;
        const long long plane = (long long)H * W;
        const long long xbase = ((long long)id.b * p.C + id.c) * D * plane;
        const long long zbase = ((long long)id.b * p.C + id.c) * SC * D * plane;
        const float *hw = p.h + (long long)id.c * SC * KT;
        const float *bias = p.bias ? p.bias + id.c * SC : nullptr;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;

        auto load_plane = [&](State &st, int k) {
            if (!st.active) return;
            const bool in = k >= 0 && k < D;
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S, row = r0 - PH + j;
                float vx = 0.f, vt = 0.f, vg = 0.f;
                if (in && j < TH + 2 * PH && row >= 0 && row < H) {
                    const long long o = xbase + (long long)k * plane + (long long)row * W + st.col;
                    vx = Elem<T>::load(p.x + o);
                    vt = Elem<T>::load(p.t1 + o);
                    vg = Elem<T>::load(p.gt1 + o);
                }
                st.px[n] = vx;
                st.pt[n] = vt;
                st.pg[n] = vg;
            }
        };
        auto store_plane = [&](State &st, int k) {
            if (!st.active) return;
            const int slot = wrap(k % XR, XR);
#pragma unroll
            for (int n = 0; n < NXR; ++n) {
                const int j = st.strip + n * S;
                if (j < TH + 2 * PH) {
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
#pragma unroll
            for (int i = 0; i < SC; ++i) {
                st.gbacc[i] = 0.f;
#pragma unroll
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + PD; ++k) {
            ex.each([&](State &st, int) {
                store_plane(st, k);
                load_plane(st, k + 1);
            });
            ex.sync();

            const int j0 = k - PD;
            ex.each([&](State &st, int) {
                if (!st.active || j0 < 0) return;
                float sv[SC][RH], gv[SC][RH];
                bool pos[SC][RH];
#pragma unroll
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
#pragma unroll
                    for (int i = 0; i < SC; ++i) {
                        float s = 0.f, g = 0.f;
                        bool keep = false;
                        if (row < H) {
                            const long long o = zbase + ((long long)i * D + j0) * plane +
                                                (long long)row * W + st.col;
                            s = Elem<T>::load(p.z + o) + (bias ? bias[i] : 0.f);
                            keep = p.relu ? s > 0.f : true;
                            if (p.relu) s = s > 0.f ? s : 0.f;
                            g = Elem<T>::load(p.gout + o);
                        }
                        sv[i][r] = s;
                        gv[i][r] = g;
                        pos[i][r] = keep;
                    }
                }
                float an[SC][RH], ad[SC][RH], ag[SC][RH];
#pragma unroll
                for (int i = 0; i < SC; ++i)
#pragma unroll
                    for (int r = 0; r < RH; ++r) an[i][r] = ad[i][r] = ag[i][r] = 0.f;
#pragma unroll
                for (int td = 0; td < KD; ++td) {
                    const int slot = wrap((j0 + PD - td) % XR, XR);
#pragma unroll
                    for (int q = 0; q < RH + 2 * PH; ++q)
#pragma unroll
                        for (int tw = 0; tw < KW; ++tw) {
                            const int o = (slot * RX + st.strip * RH + q) * P + st.col + 2 * PW - tw;
                            const float vx = ex.ld(off_x + o), vt = ex.ld(off_t + o), vg = ex.ld(off_g + o);
#pragma unroll
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 * PH + th;
                                if (rr < 0 || rr >= RH) continue;
#pragma unroll
                                for (int i = 0; i < SC; ++i) {
                                    const float wv = hw[((i * KD + td) * KH + th) * KW + tw];
                                    an[i][rr] += vx * wv;
                                    ad[i][rr] += vt * wv;
                                    ag[i][rr] += vg * wv;
                                    if (p.need_gh) st.gacc[i][(td * KH + th) * KW + tw] += sv[i][rr] * vg;
                                }
                            }
                        }
                }
#pragma unroll
                for (int r = 0; r < RH; ++r) {
                    const int row = r0 + st.strip * RH + r;
                    if (row >= H) continue;
#pragma unroll
                    for (int i = 0; i < SC; ++i) {
                        float v = gv[i][r] * (an[i][r] + p.eps) * fast_rcp(ad[i][r] + p.eps) + ag[i][r];
                        if (!pos[i][r]) v = 0.f;
                        st.gbacc[i] += v;
                        if (p.gz)
                            Elem<T>::store(p.gz + zbase + ((long long)i * D + j0) * plane +
                                               (long long)row * W + st.col, v);
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
