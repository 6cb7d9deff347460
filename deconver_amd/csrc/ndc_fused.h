// Fused, LDS-tiled kernels of the NDC update for depthwise filters (m = 1).
//
// Work decomposition (all three kernels):
//   - one workgroup owns one (sample, channel) volume and a band of TH = S*RH output rows
//     over the FULL width W, and marches along the slowest spatial axis ("planes", k);
//   - lanes run along W (coalesced global traffic, conflict-free LDS rows); a thread owns a
//     register tile of RH consecutive rows x RW consecutive columns, and moves its RW
//     columns with one global access per row (32-bit for bf16 pairs, 64-bit for fp32);
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
    int NT;      // threads per workgroup (multiple of 64, >= S*CPW)
    int TH;      // output rows per workgroup
    int ntile;   // row bands per volume
    int P;       // LDS row pitch in words
    int PL;      // zero words to the left of column 0 in an LDS row (>= PW)
    int CPW;     // column groups per row = W / RW
    int nseg;    // segments of the marching axis per volume (each its own workgroup)
    int SEG;     // planes per segment
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

// S strips of RH rows, RW columns per thread; S >= 2*PH so that the halo rows fit the
// fixed per-thread bounds
static inline bool make_tile(const March &m, int RH, int RW, int target_threads, Tile &t,
                             int min_strips = 0)
{
    const int PH = m.KH / 2, PW = m.KW / 2;
    if (m.W % RW) return false;
    const int cpw = m.W / RW;
    if (cpw > kMaxThreads) return false;
    int smin = PH > 0 ? 2 * PH : 1;
    if (smin < min_strips) smin = min_strips;
    int s = target_threads / cpw;
    const int srows = (m.H + RH - 1) / RH;
    if (s > srows) s = srows;
    if (s < smin) s = smin;
    if (s * cpw > kMaxThreads) return false;
    t.S = s;
    t.CPW = cpw;
    t.NT = round_up(s * cpw, 64);
    t.TH = s * RH;
    t.ntile = (m.H + t.TH - 1) / t.TH;
    // PW zero words left of column 0: a thread's window (its RW columns and PW either side)
    // then starts at its own first column, an even word when RW = 2
    t.PL = PW;
    t.P = round_up(t.PL + m.W + PW, RW);
    t.nseg = 1;
    t.SEG = m.D;
    return true;
}

// Split the marching axis so that a launch has enough wavefronts to fill the chip: a
// workgroup that owns planes [d0, d1) marches over them plus 2*PD warm-up planes on each
// side (whose outputs its neighbours own), so segments are kept >= 16*PD planes long.
// target: wavefronts the launch should have (about the number resident at once: more segments
// than that only add warm-up planes)
static inline void split_march(const March &m, long long blocks, Tile &t, long long target)
{
    const int PD = m.KD / 2;
    const long long waves = blocks * (t.NT / 64);
#ifndef NDC_MIN_SEG
#define NDC_MIN_SEG 4
#endif
    const int min_seg = PD > 0 ? NDC_MIN_SEG * PD : m.D;
    if (waves >= target || m.D < 2 * min_seg) return;
    long long want = (target + waves - 1) / waves;
    const int max_seg = m.D / min_seg;
    if (want > max_seg) want = max_seg;
    if (want < 2) return;
    t.SEG = round_up((m.D + (int)want - 1) / (int)want, 2);
    t.nseg = (m.D + t.SEG - 1) / t.SEG;
}

// ------------------------------------------------------------------ parameters

template <typename T> struct FwdParams {
    const T *x, *z;
    const float *h, *bias;
    const float *wtab;   // packed bf16 tap tables (bf16 dot2 kernels only)
    T *out, *t1;
    T *s_over_den, *ratio;   // optional: s/(A(t1)+eps) and (A(x)+eps)/(A(t1)+eps), shape of out
    int B, C, D, H, W;
    int relu;
    float eps;
    Tile t;
};

template <typename T> struct BwdParams {
    const T *x, *z, *t1, *gout;
    const T *s_over_den, *ratio;   // optional: what the forward call saved (both or neither)
    const float *h, *bias;
    const float *wtab;   // packed bf16 tap tables (bf16 dot2 kernels only)
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
    int d0, d1;   // planes [d0, d1) of the marching axis whose outputs this workgroup owns
};

// block_id = ((b * C + c) * nseg + segment) * ntile + row band
NDC_HD BlockId decode_block(int block_id, int C, const Tile &t, int D)
{
    BlockId id;
    const int tile = block_id % t.ntile;
    const int rest = block_id / t.ntile;
    const int seg = rest % t.nseg;
    const int bc = rest / t.nseg;
    id.b = bc / C;
    id.c = bc % C;
    id.r0 = tile * t.TH;
    id.d0 = seg * t.SEG;
    id.d1 = id.d0 + t.SEG < D ? id.d0 + t.SEG : D;
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

// NW staged words from `at`.  RW = 2: the window starts at an even word (see make_tile) and
// is read two words at a time.
template <int NW, int RW, class Exec> NDC_D void read_window(Exec &ex, int at, float (&v)[NW])
{
    if constexpr (RW == 2 && NW % 2 == 0) {
        NDC_UNROLL
        for (int u = 0; u < NW; u += 2) {
            float pair[2];
            ex.ld2(at + u, pair);
            v[u] = pair[0];
            v[u + 1] = pair[1];
        }
    } else {
        NDC_UNROLL
        for (int u = 0; u < NW; ++u) v[u] = ex.ld(at + u);
    }
}

// One K-type pass over an NR x RW register tile of outputs.  `base` addresses, in a staged
// plane of ONE source channel, the word (first input row, first own column - PW); input
// rows base .. base + NR + KH - 2 feed the NR output rows and every tap plane jd of the KD
// pending output planes.  w = taps of that source channel in (KD, KH, KW) order.
//
// PIPE (here and in a_plane): the LDS words of a row are read one row ahead of the arithmetic
// that uses them, and a scheduling fence keeps that order; for kernels that run too few
// wavefronts per SIMD to hide the LDS latency otherwise and have the registers to spare.
template <int KD, int KH, int KW, int NR, int RW, int STRIDE, bool PIPE = false, class Exec>
NDC_D void k_rows(Exec &ex, int base, int P, const float (&w)[KD * KH * KW],
                  float (*acc)[STRIDE][RW], int r_off)
{
    constexpr int NW = RW + KW - 1, NROW = NR + KH - 1;
    float vn[NW];
    if (PIPE) read_window<NW, RW>(ex, base, vn);
    NDC_UNROLL
    for (int q = 0; q < NROW; ++q) {
        float v[NW];
        if (PIPE) {
            NDC_UNROLL
            for (int u = 0; u < NW; ++u) v[u] = vn[u];
            if (q + 1 < NROW) read_window<NW, RW>(ex, base + (q + 1) * P, vn);
            ex.fence();
        } else {
            read_window<NW, RW>(ex, base + q * P, v);
        }
        NDC_UNROLL
        for (int th = 0; th < KH; ++th) {
            const int rr = q - th;
            if (rr < 0 || rr >= NR) continue;
            NDC_UNROLL
            for (int tw = 0; tw < KW; ++tw)
                NDC_UNROLL
                for (int jd = 0; jd < KD; ++jd) {
                    const float wv = w[((KD - 1 - jd) * KH + th) * KW + tw];
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) acc[jd][r_off + rr][c] += v[c + tw] * wv;
                }
        }
    }
}

// One tap plane of an A-type gather for NT tensors at once over an NR x RW register tile:
// base[t] addresses, in plane-slot form, the word (first input row, first own column - PW)
// of tensor t; wt = taps of tap plane td, indexed wt[i][th*KW + tw].
template <int KH, int KW, int KT, int SC, int NR, int RW, int NTEN, bool PIPE = false, class Exec>
NDC_D void a_plane(Exec &ex, const int (&base)[NTEN], int P, const float (&wt)[SC][KH * KW],
                   float (&acc)[NTEN][SC][NR][RW])
{
    constexpr int PH = KH / 2, NW = RW + KW - 1, NROW = NR + 2 * PH;
    float vn[NTEN][NW];
    if (PIPE) {
        NDC_UNROLL
        for (int t = 0; t < NTEN; ++t) read_window<NW, RW>(ex, base[t], vn[t]);
    }
    NDC_UNROLL
    for (int q = 0; q < NROW; ++q) {
        float v[NTEN][NW];
        if (PIPE) {
            NDC_UNROLL
            for (int t = 0; t < NTEN; ++t)
                NDC_UNROLL
                for (int u = 0; u < NW; ++u) v[t][u] = vn[t][u];
            if (q + 1 < NROW) {
                NDC_UNROLL
                for (int t = 0; t < NTEN; ++t) read_window<NW, RW>(ex, base[t] + (q + 1) * P, vn[t]);
            }
            ex.fence();
        } else {
            NDC_UNROLL
            for (int t = 0; t < NTEN; ++t) read_window<NW, RW>(ex, base[t] + q * P, v[t]);
        }
        NDC_UNROLL
        for (int th = 0; th < KH; ++th) {
            const int rr = q - 2 * PH + th;
            if (rr < 0 || rr >= NR) continue;
            NDC_UNROLL
            for (int tw = 0; tw < KW; ++tw)
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    const float wv = wt[i][th * KW + tw];
                    NDC_UNROLL
                    for (int t = 0; t < NTEN; ++t)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) acc[t][i][rr][c] += v[t][c + KW - 1 - tw] * wv;
                }
        }
    }
}

// NROWS rows of NW staged words of each of NOP operands (row n of operand t at addr(n, t)),
// handed to body(n, words); PIPE: read one row ahead of the arithmetic (see k_rows).
template <int NROWS, int NW, int NOP, bool PIPE, int RW, class Exec, class Addr, class Body>
NDC_D void stream_rows(Exec &ex, Addr addr, Body body)
{
    float vn[NOP][NW];
    if (PIPE) {
        NDC_UNROLL
        for (int t = 0; t < NOP; ++t) read_window<NW, RW>(ex, addr(0, t), vn[t]);
    }
    NDC_UNROLL
    for (int n = 0; n < NROWS; ++n) {
        float v[NOP][NW];
        if (PIPE) {
            NDC_UNROLL
            for (int t = 0; t < NOP; ++t)
                NDC_UNROLL
                for (int u = 0; u < NW; ++u) v[t][u] = vn[t][u];
            if (n + 1 < NROWS) {
                NDC_UNROLL
                for (int t = 0; t < NOP; ++t) read_window<NW, RW>(ex, addr(n + 1, t), vn[t]);
            }
            ex.fence();
        } else {
            NDC_UNROLL
            for (int t = 0; t < NOP; ++t) read_window<NW, RW>(ex, addr(n, t), v[t]);
        }
        body(n, v);
    }
}

// Filter slices, fetched into scalar registers at the top of each tap-loop iteration (keeping
// the next slice in flight as well costs more in scalar-register spills and copies than the
// load latency it hides).
template <int N> NDC_D void load_taps(UniformF src, float (&dst)[N])
{
    NDC_UNROLL
    for (int a = 0; a < N; ++a) dst[a] = src[a];
}

template <int SC, int KT, int N> NDC_D void load_plane_taps(UniformF src, float (&dst)[SC][N])
{
    NDC_UNROLL
    for (int i = 0; i < SC; ++i)
        NDC_UNROLL
        for (int a = 0; a < N; ++a) dst[i][a] = src[i * KT + a];
}

// thread coordinates shared by the three kernels
struct Lane {
    int strip, c0, active;
};

NDC_HD Lane make_lane(int tid, const Tile &t, int RW)
{
    Lane l;
    l.strip = tid / t.CPW;
    l.c0 = (tid - l.strip * t.CPW) * RW;
    l.active = l.strip < t.S;
    return l;
}

// =================================================================== forward

template <int KD_, int KH_, int KW_, int SC_, int RH_, int RW_, typename T> struct FwdKernel {
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_, RW = RW_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int XT = PH > 0 ? 1 : 0;            // one extra halo row for strips < 2*PH
    static constexpr int RHK = RH + XT;
    static constexpr int NZR = RH + (PH > 0 ? 2 : 0);    // rows of s a thread stages
    static constexpr int NXR = RH + (PH > 0 ? 1 : 0);    // rows of x a thread stages
    static constexpr int XR = KD;                        // x ring slots (filled in the scatter phase)
    typedef FwdParams<T> Params;
    typedef VecIO<T, RW> IO;

    struct State {
        Lane ln;
        int zoff[NZR], xoff[NXR], ooff[RH];   // element offsets inside one plane (rows clamped)
        unsigned zok, xok, ook;               // bit n: that row is inside the image
        float bv[SC];
        float t1acc[KD][RHK][RW];
        float pz[SC][NZR][RW];
        float px[NXR][RW];
        // LDS word offsets inside a ring slot, formed once: the word (first own row - PH, first
        // own column - PW), the word (row `strip`, first own column) and the word (halo row,
        // first own column - PW).  What is added per access (slot, row, channel) is the same in
        // every lane and stays on the scalar unit.
        int ob, so, ho;
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
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RS = rows_s(TH), RX = rows_x(TH);
        const int off_s = 0, off_x = SC * RS * P, off_t = off_x + XR * RX * P;
        const int total = off_t + KD * RX * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;   // one channel volume
        const T *xg = p.x + ((long long)id.b * p.C + id.c) * cplane;
        const T *zg = p.z + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *og = p.out + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *t1g = p.t1 ? p.t1 + ((long long)id.b * p.C + id.c) * cplane : nullptr;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;
        // owned output planes [d0, d1); the march starts 2*PD planes early so that t1 is
        // complete from plane d0 - PD on, and runs 2*PD planes past the end
        const int d0 = id.d0, d1 = id.d1;
        const int k_first = d0 - 2 * PD > 0 ? d0 - 2 * PD : 0, k_end = d1 + 2 * PD;

        // global -> registers: plane k of s (bias / ReLU applied) and plane k - PD of x.
        // Rows outside the image read a clamped address and are zeroed by a select.
        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            if (k < D) {
                const T *zk = zg + (long long)k * plane;
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n) {
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v[RW];
                        IO::load(zk + i * cplane + st.zoff[n], v);
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            float s = v[c] + st.bv[i];
                            s = floor_f(s, floor_);
                            st.pz[i][n][c] = s;
                        }
                    }
                }
            } else {
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) st.pz[i][n][c] = 0.f;
            }
            // planes outside the volume: load a clamped plane and select zero (a store in each
            // arm of a branch would push the staging registers into private memory)
            const int kx = k - PD;
            const bool xlive = kx >= 0 && kx < D;
            const T *xk = xg + (long long)clampi(kx, 0, D - 1) * plane;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                float v[RW];
                IO::load(xk + st.xoff[n], v);
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) st.px[n][c] = xlive ? v[c] : 0.f;
            }
        };

        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            // rows outside the image are never written: they keep the zeros of the set-up
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                if ((st.zok >> n) & 1u) {
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c)
                            ex.st_(st.so + (off_s + (i * RS + n * S) * P) + c, st.pz[i][n][c]);
                }
            }
        };
        // x plane k - PD into its ring slot.  Runs in the scatter phase: a barrier after the
        // gather that last read that slot, which is what lets KD slots do.
        auto store_x_plane = [&](State &st, int k) NDC_LAMBDA {
            const int slot = wrap((k - PD) % XR, XR);
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        ex.st_(st.so + (off_x + (slot * RX + n * S) * P) + c, st.px[n][c]);
                }
            }
        };

        // ---- set-up: thread coordinates, row offsets, zeroed accumulators, zeroed LDS (halo
        //      columns and never-staged rows stay zero for the whole march)
        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.ob = st.ln.strip * RH * P + PL + st.ln.c0 - PW;
            st.so = st.ln.strip * P + PL + st.ln.c0;
            st.ho = halo_row(st.ln.strip, PH, TH) * P + PL + st.ln.c0 - PW;
            st.zok = st.xok = st.ook = 0u;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RS && row >= 0 && row < H) st.zok |= 1u << n;
                st.zoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                if (row < H) st.ook |= 1u << r;
                st.ooff[r] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) st.bv[i] = p.bias ? p.bias[id.c * SC + i] : 0.f;
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) st.t1acc[a][r][c] = 0.f;
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, k_first);
        });
        ex.sync();
        ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k_first); });
        ex.sync();

        // Two barriers per plane step: the source plane of the NEXT step is staged at the end of
        // the gather phase (which does not read the source area), not in a phase of its own.
        for (int kk = k_first; kk < k_end; ++kk) {
            const int k = uniform_int(kk);   // the plane index stays on the scalar unit

            // ---- K-scatter: plane k of s feeds the KD pending planes of t1
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                store_x_plane(st, k);
                const bool extra = XT && st.ln.strip < 2 * PH;
                const int jx = halo_row(st.ln.strip, PH, TH);
                if (k < D) {
                    NDC_ROLLED
                    for (int ii = 0; ii < SC; ++ii) {
                        const int i = uniform_int(ii);
                        float wi[KT];
                        load_taps<KT>(hw + i * KT, wi);
                        k_rows<KD, KH, KW, RH, RW, RHK>(ex, st.ob + (off_s + (i * RS + PH) * P), P, wi,
                                                        st.t1acc, 0);
                        if (extra) k_rows<KD, KH, KW, 1, RW, RHK>(ex, st.ho + (off_s + i * RS * P), P, wi, st.t1acc, RH);
                    }
                }
                // plane k - PD of t1 is complete: publish it (zero outside the volume)
                const int pf = k - PD;
                const bool inplane = pf >= 0 && pf < D;
                const int tb = off_t + wrap(pf % KD, KD) * RX * P;
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r) {
                    const bool mine = r < RH || extra;
                    const int j = r < RH ? PH + st.ln.strip * RH + r : jx;
                    const int row = r0 - PH + j;
                    const bool live = inplane && row >= 0 && row < H;
                    float v[RW];
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        v[c] = live ? st.t1acc[0][r][c] : 0.f;
                        if (mine) ex.st_((r < RH ? st.ob + (tb + (PH + r) * P) : st.ho + tb) + PW + c, v[c]);
                    }
                    if (r < RH && t1g && live && pf >= d0 && pf < d1)
                        IO::store(t1g + (long long)pf * plane + st.ooff[r < RH ? r : 0], v);
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        NDC_UNROLL
                        for (int a = 0; a + 1 < KD; ++a) st.t1acc[a][r][c] = st.t1acc[a + 1][r][c];
                        st.t1acc[KD - 1][r][c] = 0.f;
                    }
                }
            });
            ex.sync();

            // ---- prefetch of the next plane, then A-gather + epilogue for plane k - 2*PD
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                load_plane(st, k + 1);
                const int j0 = k - 2 * PD;
                if (j0 < d0) {
                    store_plane(st, k + 1);
                    return;
                }
                // the thread's own source values: re-read from global (an L2 hit) rather
                // than carried in registers across 2*PD planes
                float sv[SC][RH][RW];
                const T *zk = zg + (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        IO::load(zk + i * cplane + st.ooff[r], sv[i][r]);
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            float s = sv[i][r][c] + st.bv[i];
                            s = floor_f(s, floor_);
                            sv[i][r][c] = s;
                        }
                    }
                float acc[2][SC][RH][RW];
                NDC_UNROLL
                for (int a = 0; a < 2; ++a)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) acc[a][i][r][c] = 0.f;
                NDC_ROLLED
                for (int tdd = 0; tdd < KD; ++tdd) {
                    const int td = uniform_int(tdd);
                    float wt[SC][KH * KW];
                    load_plane_taps<SC, KT, KH * KW>(hw + td * KH * KW, wt);
                    const int pl = j0 + PD - td;
                    const int base[2] = {st.ob + (off_x + wrap(pl % XR, XR) * RX * P),
                                         st.ob + (off_t + wrap(pl % KD, KD) * RX * P)};
                    a_plane<KH, KW, KT, SC, RH, RW, 2>(ex, base, P, wt, acc);
                }
                T *ok_ = og + (long long)j0 * plane;
                T *dk_ = p.s_over_den ? p.s_over_den + (og - p.out) + (long long)j0 * plane : nullptr;
                T *rk_ = p.ratio ? p.ratio + (og - p.out) + (long long)j0 * plane : nullptr;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (!((st.ook >> r) & 1u)) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v[RW], rd[RW], rt[RW];
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            const float inv = fast_rcp(acc[1][i][r][c] + eps);
                            rd[c] = sv[i][r][c] * inv;
                            rt[c] = (acc[0][i][r][c] + eps) * inv;
                            v[c] = sv[i][r][c] * rt[c];
                        }
                        IO::store(ok_ + i * cplane + st.ooff[r], v);
                        if (dk_) {
                            IO::store(dk_ + i * cplane + st.ooff[r], rd);
                            IO::store(rk_ + i * cplane + st.ooff[r], rt);
                        }
                    }
                }
                store_plane(st, k + 1);
            });
            ex.sync();
        }
    }
};

// =================================================================== backward, pass 1

// SAVED: the call brings the forward's s/d and n/d, so gn = g (s/d), gd = -gn (n/d) are
// elementwise (z is not read, n and d are not re-gathered); the x / t1 rings then serve the
// filter-gradient terms only.
template <int KD_, int KH_, int KW_, int SC_, int RH_, int RW_, typename T, bool SAVED_ = false>
struct Bwd1Kernel {
    static constexpr bool SAVED = SAVED_;
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_, RW = RW_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int XT = PH > 0 ? 1 : 0;
    static constexpr int NXR = RH + (PH > 0 ? 2 : 0);   // rows of x/t1 a thread stages
    static constexpr int XR = KD + 1;
    static constexpr int NRED = SC * KT;
    typedef BwdParams<T> Params;
    typedef VecIO<T, RW> IO;

    struct State {
        Lane ln;
        int xoff[NXR], ooff[RH];
        unsigned xok, ook;
        float bv[SC];
        float gacc[SC][KT];          // A-side filter-gradient terms
        // LDS word offsets inside a ring slot, formed once: the word (first own row - PH of an
        // x / t1 slot's rows, first own column - PW), the word (row `strip`, first own column)
        // and the word (halo row of a gn / gd plane, first own column); what is added per access
        // (slot, row, channel) is the same in every lane and stays on the scalar unit
        int ob, so, ho;
        float accx[KD][RH][RW];      // pending planes of gx
        float acct[KD][RH][RW];      // pending planes of gt1
        float px[NXR][RW], pt[NXR][RW];
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

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH), RG = rows_g(TH);
        const int off_x = 0, off_t = XR * RX * P, off_g = 2 * XR * RX * P;
        const int total = off_g + 2 * SC * RG * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const T *xg = p.x + cbase, *t1g = p.t1 + cbase;
        const T *zg = p.z + cbase * SC, *gg = p.gout + cbase * SC;
        const T *dg = SAVED ? p.s_over_den + cbase * SC : nullptr;
        const T *rg = SAVED ? p.ratio + cbase * SC : nullptr;
        T *gxg = p.gx ? p.gx + cbase : nullptr;
        T *gt1g = p.gt1 + cbase;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;
        const int need_gh = p.need_gh;
        // owned output planes [d0, d1); gn / gd are needed PD planes beyond them on each side
        // and the x / t1 rings another PD planes beyond that
        const int d0 = id.d0, d1 = id.d1;
        const int k_first = d0 - 2 * PD > 0 ? d0 - 2 * PD : 0, k_end = d1 + 2 * PD;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            // planes past the end: load the last plane and select zero (a store in each arm of
            // a branch would push the staging registers into private memory)
            const bool live = k < D;
            const long long ko = (long long)clampi(k, 0, D - 1) * plane;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                float vx[RW], vt[RW];
                IO::load(xg + ko + st.xoff[n], vx);
                IO::load(t1g + ko + st.xoff[n], vt);
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) {
                    st.px[n][c] = live ? vx[c] : 0.f;
                    st.pt[n][c] = live ? vt[c] : 0.f;
                }
            }
        };
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int slot = wrap(k % XR, XR);
            // rows outside the image are never written: they keep the zeros of the set-up
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        const int o = st.so + (slot * RX + n * S) * P + c;
                        ex.st_(off_x + o, st.px[n][c]);
                        ex.st_(off_t + o, st.pt[n][c]);
                    }
                }
            }
        };

        // gn, gd of NR rows starting at gn/gd tile row j (image row r0 - PH + j): computed,
        // published to LDS, and returned in acc[0] / acc[1]
        // lo: LDS word offset of (tile row j, first own column) inside a plane
        auto gn_gd_rows = [&](State &st, int j1, int j, int lo, auto nr_tag,
                              float (&acc)[2][SC][decltype(nr_tag)::value][RW]) NDC_LAMBDA {
            constexpr int NR = decltype(nr_tag)::value;
            float sv[SC][NR][RW], gv[SC][NR][RW];
            const long long ko = (long long)j1 * plane;
            NDC_UNROLL
            for (int r = 0; r < NR; ++r) {
                const int row = r0 - PH + j + r;
                const bool ok = row >= 0 && row < H;
                const int o = clampi(row, 0, H - 1) * W + st.ln.c0;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    IO::load(gg + i * cplane + ko + o, gv[i][r]);
                    if (SAVED) {
                        // sv <- s/d, acc[0] <- n/d (as saved by the forward)
                        IO::load(dg + i * cplane + ko + o, sv[i][r]);
                        IO::load(rg + i * cplane + ko + o, acc[0][i][r]);
                    } else {
                        IO::load(zg + i * cplane + ko + o, sv[i][r]);
                    }
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        if (!SAVED) {
                            float s = sv[i][r][c] + st.bv[i];
                            s = floor_f(s, floor_);
                            sv[i][r][c] = s;
                        }
                        gv[i][r][c] = ok ? gv[i][r][c] : 0.f;
                    }
                }
            }
            if (!SAVED) {
                NDC_UNROLL
                for (int a = 0; a < 2; ++a)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int r = 0; r < NR; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) acc[a][i][r][c] = 0.f;
                NDC_ROLLED
                for (int tdd = 0; tdd < KD; ++tdd) {
                    const int td = uniform_int(tdd);
                    float wt[SC][KH * KW];
                    load_plane_taps<SC, KT, KH * KW>(hw + td * KH * KW, wt);
                    const int slot = wrap((j1 + PD - td) % XR, XR);
                    const int ob = lo - PW + slot * RX * P;
                    const int base[2] = {off_x + ob, off_t + ob};
                    a_plane<KH, KW, KT, SC, NR, RW, 2>(ex, base, P, wt, acc);
                }
            }
            NDC_UNROLL
            for (int r = 0; r < NR; ++r)
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        float gn, gd;
                        if (SAVED) {
                            gn = gv[i][r][c] * sv[i][r][c];
                            gd = -(gn * acc[0][i][r][c]);
                        } else {
                            const float inv = fast_rcp(acc[1][i][r][c] + eps);
                            gn = gv[i][r][c] * sv[i][r][c] * inv;
                            gd = -(gn * (acc[0][i][r][c] + eps)) * inv;
                        }
                        ex.st_(lo + (off_g + (i * RG + r) * P) + c, gn);
                        ex.st_(lo + (off_g + ((SC + i) * RG + r) * P) + c, gd);
                        acc[0][i][r][c] = gn;
                        acc[1][i][r][c] = gd;
                    }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.ob = st.ln.strip * RH * P + PL + st.ln.c0 - PW;
            st.so = st.ln.strip * P + PL + st.ln.c0;
            st.ho = halo_row(st.ln.strip, PH, TH) * P + PL + st.ln.c0;
            st.xok = st.ook = 0u;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                if (row < H) st.ook |= 1u << r;
                st.ooff[r] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) {
                st.bv[i] = p.bias ? p.bias[id.c * SC + i] : 0.f;
                NDC_UNROLL
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
            }
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) st.accx[a][r][c] = st.acct[a][r][c] = 0.f;
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, k_first);
        });
        ex.sync();
        ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k_first); });
        ex.sync();

        // Two barriers per plane step: the (x, t1) plane of the NEXT step is staged at the end
        // of the scatter phase, into the ring slot that no phase of this step reads.
        for (int kk = k_first; kk < k_end; ++kk) {
            const int k = uniform_int(kk);   // the plane index stays on the scalar unit

            // ---- gather: gn, gd of plane k - PD on the band plus PH halo rows each side
            const int j1 = k - PD;
            const bool live1 = j1 >= 0 && j1 < D && j1 >= d0 - PD;
            const bool own1 = j1 >= d0 && j1 < d1;   // filter-gradient terms: owned planes only
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active || !live1) return;
                {
                    float acc[2][SC][RH][RW];
                    const int j = PH + st.ln.strip * RH;
                    gn_gd_rows(st, j1, j, st.ob + (PW + PH * P), IntTag<RH>(), acc);
                    if (need_gh && own1) {
                        // own rows: A-side filter-gradient terms, re-reading the x / t1 windows
                        // (read ahead: for the 2x2 float32 tile this costs two spilled registers
                        // and is still 3 % faster)
                        constexpr int NQ = RH + 2 * PH;
                        stream_rows<KD * NQ, RW + KW - 1, 2, (KH > 1 && SAVED), RW>(
                            ex,
                            [&](int n, int t) NDC_LAMBDA {
                                const int td = n / NQ, q = n % NQ;
                                const int slot = wrap((j1 + PD - td) % XR, XR);
                                return st.ob + ((t ? off_t : off_x) + (slot * RX + PH + q) * P);
                            },
                            [&](int n, const float (&v)[2][RW + KW - 1]) NDC_LAMBDA {
                                const int td = n / NQ, q = n % NQ;
                                NDC_UNROLL
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - 2 * PH + th;
                                    if (rr >= 0 && rr < RH) {
                                        NDC_UNROLL
                                        for (int tw = 0; tw < KW; ++tw)
                                            NDC_UNROLL
                                            for (int i = 0; i < SC; ++i)
                                                NDC_UNROLL
                                                for (int c = 0; c < RW; ++c) {
                                                    // two fused multiply-adds (a sum of two
                                                    // products added on costs a third instruction)
                                                    float &ga = st.gacc[i][(td * KH + th) * KW + tw];
                                                    ga += acc[0][i][rr][c] * v[0][c + KW - 1 - tw];
                                                    ga += acc[1][i][rr][c] * v[1][c + KW - 1 - tw];
                                                }
                                    }
                                }
                            });
                    }
                }
                if (XT && st.ln.strip < 2 * PH) {
                    float acc[2][SC][1][RW];
                    gn_gd_rows(st, j1, halo_row(st.ln.strip, PH, TH), st.ho, IntTag<1>(), acc);
                }
            });
            ex.sync();

            // ---- prefetch, then scatter: plane k - PD of gn/gd feeds pending planes of gx / gt1
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                load_plane(st, k + 1);
                if (live1) {
                    NDC_ROLLED
                    for (int ii = 0; ii < SC; ++ii) {
                        const int i = uniform_int(ii);
                        float wi[KT];
                        load_taps<KT>(hw + i * KT, wi);
                        const int gb_ = st.ob + off_g;
                        k_rows<KD, KH, KW, RH, RW, RH, (KH > 1 && SAVED)>(ex, gb_ + i * RG * P, P, wi, st.accx, 0);
                        k_rows<KD, KH, KW, RH, RW, RH, (KH > 1 && SAVED)>(ex, gb_ + (SC + i) * RG * P, P, wi, st.acct, 0);
                    }
                }
                const int pf = k - 2 * PD;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (pf >= d0 && ((st.ook >> r) & 1u)) {
                        const long long o = (long long)pf * plane + st.ooff[r];
                        if (gxg) IO::store(gxg + o, st.accx[0][r]);
                        IO::store(gt1g + o, st.acct[0][r]);
                    }
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        NDC_UNROLL
                        for (int a = 0; a + 1 < KD; ++a) {
                            st.accx[a][r][c] = st.accx[a + 1][r][c];
                            st.acct[a][r][c] = st.acct[a + 1][r][c];
                        }
                        st.accx[KD - 1][r][c] = 0.f;
                        st.acct[KD - 1][r][c] = 0.f;
                    }
                }
                store_plane(st, k + 1);
            });
            ex.sync();
        }

        if (need_gh) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            ex.template block_reduce<NRED>(
                [](State &st, int i) NDC_LAMBDA { return st.gacc[i / KT][i % KT]; },
                [&](int i, float v) NDC_LAMBDA { dst[i] = v; });
        }
    }
};

// =================================================================== backward, pass 2

// SAVED: gz = [s > 0] (g (n/d) + A(gt1)) with the forward's n/d: only the gt1 ring is kept.
template <int KD_, int KH_, int KW_, int SC_, int RH_, int RW_, typename T, bool SAVED_ = false>
struct Bwd2Kernel {
    static constexpr bool SAVED = SAVED_;
    static constexpr int NA = SAVED ? 1 : 3;   // gathered operands: (x, t1,) gt1
    static constexpr int KD = KD_, KH = KH_, KW = KW_, SC = SC_, RH = RH_, RW = RW_;
    static constexpr int PD = KD / 2, PH = KH / 2, PW = KW / 2, KT = KD * KH * KW;
    static constexpr int NXR = RH + (PH > 0 ? 1 : 0);
    static constexpr int XR = KD + 1;
    static constexpr int NRED = SC * KT + SC;
    typedef BwdParams<T> Params;
    typedef VecIO<T, RW> IO;

    struct State {
        Lane ln;
        int xoff[NXR], ooff[RH];
        unsigned xok, ook;
        float bv[SC];
        float gacc[SC][KT];   // K-side filter-gradient term
        // LDS word offsets inside a ring slot, formed once: the word (first own row - PH, first
        // own column - PW) and the word (row `strip`, first own column); what is added per
        // access (slot, row) is the same in every lane and stays on the scalar unit
        int ob, so;
        float gbacc[SC];
        float px[NXR][RW], pt[NXR][RW], pg[NXR][RW];
    };

    static NDC_HD int rows_x(int TH) { return TH + 2 * PH; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = NA * XR * rows_x(t.TH) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH);
        const int off_x = 0, off_t = XR * RX * P, off_g = SAVED ? 0 : 2 * XR * RX * P;
        const int total = NA * XR * RX * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const T *xg = p.x + cbase, *t1g = p.t1 + cbase, *gt1g = p.gt1 + cbase;
        const T *zg = p.z + cbase * SC, *gg = p.gout + cbase * SC;
        const T *rg = SAVED ? p.ratio + cbase * SC : nullptr;
        T *gzg = p.gz ? p.gz + cbase * SC : nullptr;
        UniformF hw = as_uniform(p.h + (long long)id.c * SC * KT);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;
        const int need_gh = p.need_gh;
        // owned output planes [d0, d1); the rings need PD planes of lead-in and lead-out
        const int d0 = id.d0, d1 = id.d1;
        const int k_first = d0 - PD > 0 ? d0 - PD : 0, k_end = d1 + PD;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            // planes past the end: load the last plane and select zero (a store in each arm of
            // a branch would push the staging registers into private memory)
            const bool live = k < D;
            const long long ko = (long long)clampi(k, 0, D - 1) * plane;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                float vx[RW], vt[RW], vg[RW];
                if (!SAVED) {
                    IO::load(xg + ko + st.xoff[n], vx);
                    IO::load(t1g + ko + st.xoff[n], vt);
                }
                IO::load(gt1g + ko + st.xoff[n], vg);
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) {
                    st.px[n][c] = (!SAVED && live) ? vx[c] : 0.f;
                    st.pt[n][c] = (!SAVED && live) ? vt[c] : 0.f;
                    st.pg[n][c] = live ? vg[c] : 0.f;
                }
            }
        };
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int slot = wrap(k % XR, XR);
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        const int o = st.so + (slot * RX + n * S) * P + c;
                        if (!SAVED) {
                            ex.st_(off_x + o, st.px[n][c]);
                            ex.st_(off_t + o, st.pt[n][c]);
                        }
                        ex.st_(off_g + o, st.pg[n][c]);
                    }
                }
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.ob = st.ln.strip * RH * P + PL + st.ln.c0 - PW;
            st.so = st.ln.strip * P + PL + st.ln.c0;
            st.xok = st.ook = 0u;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                if (row < H) st.ook |= 1u << r;
                st.ooff[r] = clampi(row, 0, H - 1) * W + st.ln.c0;
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) {
                st.bv[i] = p.bias ? p.bias[id.c * SC + i] : 0.f;
                st.gbacc[i] = 0.f;
                NDC_UNROLL
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, k_first);
        });
        ex.sync();

        for (int kk = k_first; kk < k_end; ++kk) {
            const int k = uniform_int(kk);   // the plane index stays on the scalar unit
            ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k); });
            ex.sync();

            const int j0 = k - PD;
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                load_plane(st, k + 1);
                if (j0 < d0) return;
                float sv[SC][RH][RW], gv[SC][RH][RW], rv[SC][RH][RW];
                const long long ko = (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    const bool ok = (st.ook >> r) & 1u;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        IO::load(zg + i * cplane + ko + st.ooff[r], sv[i][r]);
                        IO::load(gg + i * cplane + ko + st.ooff[r], gv[i][r]);
                        if (SAVED) {
                            IO::load(rg + i * cplane + ko + st.ooff[r], rv[i][r]);
                        } else {
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) rv[i][r][c] = 0.f;
                        }
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            // with the ReLU on, s <= 0 marks a masked element
                            float s = sv[i][r][c] + st.bv[i];
                            s = floor_f(s, floor_);
                            sv[i][r][c] = ok ? s : 0.f;
                            gv[i][r][c] = ok ? gv[i][r][c] : 0.f;
                        }
                    }
                }
                float acc[NA][SC][RH][RW];
                NDC_UNROLL
                for (int a = 0; a < NA; ++a)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) acc[a][i][r][c] = 0.f;
                NDC_ROLLED
                for (int tdd = 0; tdd < KD; ++tdd) {
                    const int td = uniform_int(tdd);
                    float wt[SC][KH * KW];
                    load_plane_taps<SC, KT, KH * KW>(hw + td * KH * KW, wt);
                    const int slot = wrap((j0 + PD - td) % XR, XR);
                    const int ob = st.ob + slot * RX * P;
                    int base[NA];
                    base[NA - 1] = off_g + ob;
                    if (!SAVED) {
                        base[0] = off_x + ob;
                        base[NA > 1 ? 1 : 0] = off_t + ob;
                    }
                    a_plane<KH, KW, KT, SC, RH, RW, NA, (KH > 1 && SAVED)>(ex, base, P, wt, acc);
                }
                if (need_gh) {
                    // K-side filter-gradient term: re-read the gt1 window
                    constexpr int NQ = RH + 2 * PH;
                    stream_rows<KD * NQ, RW + KW - 1, 1, (KH > 1 && SAVED), RW>(
                        ex,
                        [&](int n, int) NDC_LAMBDA {
                            const int td = n / NQ, q = n % NQ;
                            const int slot = wrap((j0 + PD - td) % XR, XR);
                            return st.ob + (off_g + (slot * RX + q) * P);
                        },
                        [&](int n, const float (&v)[1][RW + KW - 1]) NDC_LAMBDA {
                            const int td = n / NQ, q = n % NQ;
                            NDC_UNROLL
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 * PH + th;
                                if (rr >= 0 && rr < RH) {
                                    NDC_UNROLL
                                    for (int tw = 0; tw < KW; ++tw)
                                        NDC_UNROLL
                                        for (int i = 0; i < SC; ++i)
                                            NDC_UNROLL
                                            for (int c = 0; c < RW; ++c)
                                                st.gacc[i][(td * KH + th) * KW + tw] +=
                                                    sv[i][rr][c] * v[0][c + KW - 1 - tw];
                                }
                            }
                        });
                }
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (!((st.ook >> r) & 1u)) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v[RW];
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            float gzv;
                            if (SAVED)
                                gzv = gv[i][r][c] * rv[i][r][c] + acc[NA - 1][i][r][c];
                            else
                                gzv = gv[i][r][c] * (acc[0][i][r][c] + eps) *
                                          fast_rcp(acc[NA > 1 ? 1 : 0][i][r][c] + eps) +
                                      acc[NA - 1][i][r][c];
                            if (p.relu && sv[i][r][c] <= 0.f) gzv = 0.f;   // a NaN passes
                            st.gbacc[i] += gzv;
                            v[c] = gzv;
                        }
                        if (gzg) IO::store(gzg + i * cplane + ko + st.ooff[r], v);
                    }
                }
            });
        }

        if (p.need_gh || p.need_gb) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            ex.template block_reduce<NRED>(
                [](State &st, int i) NDC_LAMBDA {
                    return i < SC * KT ? st.gacc[(i < SC * KT ? i : 0) / KT][i % KT]
                                       : st.gbacc[i >= SC * KT ? i - SC * KT : 0];
                },
                [&](int i, float v) NDC_LAMBDA { dst[i] = v; });
        }
    }
};

}  // namespace fused
}  // namespace ndc
