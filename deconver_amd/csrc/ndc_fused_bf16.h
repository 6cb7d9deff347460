// bfloat16 variants of the fused kernels for the 3x3x3, SC = 4 depthwise geometry, built on
// v_dot2c_f32_bf16 (two bf16 MACs per lane-instruction, float32 accumulate, same issue
// rate as an fp32 FMA that takes its tap from a scalar register).  Same work decomposition, rings and march as ndc_fused.h; what
// changes is the LDS word format and the tap loops:
//
//   K-type applications (4 -> 1 channels) pair CHANNELS: the staged source is kept as two
//     words per voxel, (s0, s1) and (s2, s3), and multiplied with the packed tap pairs
//     (h0, h1)[tau], (h2, h3)[tau]: 2 dot2 per tap instead of 4 FMAs.
//   A-type applications (1 -> 4 channels) pair PLANES: ring slot m of a single-channel
//     operand v holds the word (v[m], v[m+1]) per voxel, so that
//       A(v)[i, j] = sum_{th,tw}  P[j-1] . (h[i,2,th,tw], h[i,1,th,tw])
//                               + P[j]   . (0,           h[i,0,th,tw])
//     : 2 dot2 per (th, tw) instead of 3 FMAs.  The producer of plane m+1 completes word m
//     from the value of plane m it kept in a register.
//     The forward and the kept-ratio pass 2 replace the half-empty second term by COLUMN
//     pairs of plane j+1, which arrive from global memory (or leave for it) in that form:
//     with Q[c] = (v[2c], v[2c+1]) of plane j+1, per input row
//       column 2c  :  Q[c] . (h1, h0) + Q[c-1] . (0,  h2)        h_tw = h[i,0,th,tw]
//       column 2c+1:  Q[c] . (h2, h1) + Q[c+1] . (h0, 0)
//     : 4 dot2 per column pair for the 6 products of a tap row, 15 instead of 18 dot2 per
//     output voxel and source channel.
//   The filter-gradient terms pair OPERANDS: (gn_i, gd_i) . (x, t1)[neighbour] in pass 1,
//     and (s_i[j-1], s_i[j]) . (gt1[m], gt1[m+1])[neighbour] every second plane in pass 2.
//
// Taps are rounded to bfloat16 for the multiplications (the gradient that is returned is
// the one with respect to the float32 filter, as under bf16 autocast); accumulation,
// numerator/denominator arithmetic and all reductions stay float32.  The packed tap tables
// are prepared by a small kernel into the call's workspace: per channel
//   WK[p][tau]        = (h[2p][tau], h[2p+1][tau])            p = 0, 1       54 words
//   WA[s][i][th][tw]  = s = 0: (h[i][2][th][tw], h[i][1][th][tw])
//                       s = 1: (0,               h[i][0][th][tw])             72 words
//   WQ[th][i][n]      = n = 0: (h1, h0)  1: (0, h2)  2: (h2, h1)  3: (h0, 0),
//                       h_tw = h[i][0][th][tw]                                  48 words
//   WM[m][th][tw]     = rows of the 4x4 tap matrices of the matrix-instruction kernels
//                       (ndc_fused_mfma.h): the four source channels' taps of tap plane
//                       2 - m, (h[0], h[1]) then (h[2], h[3]); m = 3: zeros        72 words
//   WG[i][td][th]     = rows of the tap matrices of the A-type applications there: the
//                       tap row against a 4-column window, (h2, h1) then (h0, 0),
//                       h_tw = h[i][td][th][tw]                                     72 words
#pragma once

#include "ndc_fused.h"

namespace ndc {
namespace fused {

static const int kTabWK = 0, kTabWA = 54, kTabWQ = 126, kTabWM = 174, kTabWG = 246;
static const int kTabWords = 318;   // packed tap words per channel (54 WK + 72 WA + 48 WQ + 72 WM + 72 WG)

// idx over C * kTabWords
NDC_HD void prep_tables(long long idx, const float *h, float *tab)
{
    const int c = (int)(idx / kTabWords), e = (int)(idx % kTabWords);
    const float *hc = h + (long long)c * 4 * 27;
    uint32_t w;
    if (e < 54) {
        const int p = e / 27, tau = e % 27;
        w = pack_bf16x2(hc[(2 * p) * 27 + tau], hc[(2 * p + 1) * 27 + tau]);
    } else if (e < kTabWQ) {
        const int r = e - 54, s = r / 36, i = (r % 36) / 9, t9 = r % 9;
        w = s == 0 ? pack_bf16x2(hc[i * 27 + 2 * 9 + t9], hc[i * 27 + 1 * 9 + t9])
                   : pack_bf16x2(0.f, hc[i * 27 + t9]);
    } else if (e < kTabWM) {
        const int r = e - kTabWQ, th = r / 16, i = (r % 16) / 4, n = r % 4;
        const float *ht = hc + i * 27 + th * 3;   // the tap row h[i][0][th][0..2]
        w = n == 0 ? pack_bf16x2(ht[1], ht[0]) : n == 1 ? pack_bf16x2(0.f, ht[2])
          : n == 2 ? pack_bf16x2(ht[2], ht[1]) : pack_bf16x2(ht[0], 0.f);
    } else if (e < kTabWG) {
        const int r = e - kTabWM, m = r / 18, t9 = (r % 18) / 2, half = r % 2;
        const int tau = (2 - m) * 9 + t9;
        w = m == 3 ? 0u : pack_bf16x2(hc[(2 * half) * 27 + tau], hc[(2 * half + 1) * 27 + tau]);
    } else {
        const int r = e - kTabWG, i = r / 18, t9 = (r % 18) / 2, half = r % 2;
        const float *ht = hc + i * 27 + t9 * 3;   // the tap row h[i][td][th][0..2]
        w = half == 0 ? pack_bf16x2(ht[2], ht[1]) : pack_bf16x2(ht[0], 0.f);
    }
    tab[idx] = bits_to_float(w);
}

// (lo of a, lo of b) and (hi of a, hi of b) of two packed pairs: one v_perm_b32 each
NDC_HD uint32_t zip_lo(uint32_t a, uint32_t b)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_perm(b, a, 0x05040100u);
#else
    return (a & 0xffffu) | (b << 16);
#endif
}
NDC_HD uint32_t zip_hi(uint32_t a, uint32_t b)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_perm(b, a, 0x07060302u);
#else
    return (a >> 16) | (b & 0xffff0000u);
#endif
}
NDC_HD float bf_lo(uint32_t w) { return bits_to_float(w << 16); }
NDC_HD float bf_hi(uint32_t w) { return bits_to_float(w & 0xffff0000u); }

// NW staged words from `at`; four at a time where NW = 4 (the word index of every such read
// is even: a thread's window starts at its own first column, see make_tile)
template <int NW, class Exec> NDC_D void read_words(Exec &ex, int at, uint32_t (&v)[NW])
{
    if constexpr (NW == 4) {
        ex.ld4(at, v);
    } else {
        NDC_UNROLL
        for (int u = 0; u < NW; ++u) v[u] = float_to_bits(ex.ld(at + u));
    }
}

// K-type pass over an NR x RW tile for ONE channel pair: words (s_2p, s_2p+1) staged at
// `base` (first input row, first own column - 1); w = WK[p], 27 packed tap pairs.
template <int NR, int RW, int STRIDE>
NDC_D void k_row_d2(int q, const uint32_t (&v)[RW + 2], const float (&w)[27],
                    float (*acc)[STRIDE][RW], int r_off)
{
    NDC_UNROLL
    for (int th = 0; th < 3; ++th) {
        const int rr = q - th;
        if (rr >= 0 && rr < NR) {
            NDC_UNROLL
            for (int tw = 0; tw < 3; ++tw)
                NDC_UNROLL
                for (int jd = 0; jd < 3; ++jd) {
                    const uint32_t wv = float_to_bits(w[((2 - jd) * 3 + th) * 3 + tw]);
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        acc[jd][r_off + rr][c] = dot2_bf16(v[c + tw], wv, acc[jd][r_off + rr][c]);
                }
        }
    }
}

//
// PIPE (here and below): the LDS words of a row are read one row ahead of the arithmetic
// that uses them, and a scheduling fence keeps that order.  The backward kernels run two
// wavefronts per SIMD, too few to hide the LDS latency otherwise (pass 1: 0.79 -> 0.75 ms);
// the forward runs four and would lose one to the extra registers.
template <int NR, int RW, int STRIDE, bool PIPE, class Exec>
NDC_D void k_rows_d2(Exec &ex, int base, int P, const float (&w)[27], float (*acc)[STRIDE][RW],
                     int r_off)
{
    uint32_t vn[RW + 2];
    if (PIPE) read_words<RW + 2>(ex, base, vn);
    NDC_UNROLL
    for (int q = 0; q < NR + 2; ++q) {
        uint32_t v[RW + 2];
        if (PIPE) {
            NDC_UNROLL
            for (int u = 0; u < RW + 2; ++u) v[u] = vn[u];
            if (q + 1 < NR + 2) read_words<RW + 2>(ex, base + (q + 1) * P, vn);
            ex.fence();
        } else {
            read_words<RW + 2>(ex, base + q * P, v);
        }
        k_row_d2<NR, RW, STRIDE>(q, v, w, acc, r_off);
    }
}

// A-type pass over an NR x RW tile for one plane-pair slot of NTEN operands; wt = WA[s].
// FRESH: the sums start here, from `init` (what `acc` holds on entry is not read).
template <int NR, int RW, int NTEN, bool PIPE, bool FRESH = false, class Exec>
NDC_D void a_plane_d2(Exec &ex, const int (&base)[NTEN], int P, const float (&wt)[4][9],
                      float (&acc)[NTEN][4][NR][RW], float init = 0.f)
{
    uint32_t vn[NTEN][RW + 2];
    if (PIPE) {
        NDC_UNROLL
        for (int t = 0; t < NTEN; ++t) read_words<RW + 2>(ex, base[t], vn[t]);
    }
    NDC_UNROLL
    for (int q = 0; q < NR + 2; ++q) {
        uint32_t v[NTEN][RW + 2];
        if (PIPE) {
            NDC_UNROLL
            for (int t = 0; t < NTEN; ++t)
                NDC_UNROLL
                for (int u = 0; u < RW + 2; ++u) v[t][u] = vn[t][u];
            if (q + 1 < NR + 2) {
                NDC_UNROLL
                for (int t = 0; t < NTEN; ++t) read_words<RW + 2>(ex, base[t] + (q + 1) * P, vn[t]);
            }
            ex.fence();
        } else {
            NDC_UNROLL
            for (int t = 0; t < NTEN; ++t) read_words<RW + 2>(ex, base[t] + q * P, v[t]);
        }
        NDC_UNROLL
        for (int th = 0; th < 3; ++th) {
            const int rr = q - 2 + th;
            if (rr < 0 || rr >= NR) continue;
            NDC_UNROLL
            for (int tw = 0; tw < 3; ++tw)
                NDC_UNROLL
                for (int i = 0; i < 4; ++i) {
                    const uint32_t wv = float_to_bits(wt[i][th * 3 + tw]);
                    // an output row's first term comes from its first input row (q = rr: th = 2)
                    // and first column tap
                    const bool first = FRESH && th == 2 && tw == 0;
                    NDC_UNROLL
                    for (int t = 0; t < NTEN; ++t)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c)
                            acc[t][i][rr][c] = first ? dot2_bf16_from(v[t][c + 2 - tw], wv, init)
                                                     : dot2_bf16(v[t][c + 2 - tw], wv, acc[t][i][rr][c]);
                }
        }
    }
}

// The depth tap td = 0 of an A-type application (input plane j + 1) from column-pair words:
// base[t] = word (first output row - 1, own column pair - 1) of operand t's plane, staged
// with row pitch PQ; wq = WQ of the channel.  Rolled over the tap rows: 16 packed taps in
// scalar registers per iteration, NR rows of three words read for each.
template <int NR, int NTEN, class Exec>
NDC_D void a_plane_q(Exec &ex, const int (&base)[NTEN], int PQ, UniformF wq,
                     float (&acc)[NTEN][4][NR][2])
{
    NDC_ROLLED
    for (int thh = 0; thh < 3; ++thh) {
        const int th = uniform_int(thh);
        float w[16];
        load_taps<16>(wq + th * 16, w);
        NDC_UNROLL
        for (int r = 0; r < NR; ++r) {
            const int at = (r + 2 - th) * PQ;
            uint32_t v[NTEN][3];
            NDC_UNROLL
            for (int t = 0; t < NTEN; ++t)
                NDC_UNROLL
                for (int u = 0; u < 3; ++u) v[t][u] = float_to_bits(ex.ld(base[t] + at + u));
            NDC_UNROLL
            for (int i = 0; i < 4; ++i)
                NDC_UNROLL
                for (int t = 0; t < NTEN; ++t) {
                    float a0 = acc[t][i][r][0], a1 = acc[t][i][r][1];
                    a0 = dot2_bf16(v[t][1], float_to_bits(w[i * 4 + 0]), a0);
                    a1 = dot2_bf16(v[t][1], float_to_bits(w[i * 4 + 2]), a1);
                    a0 = dot2_bf16(v[t][0], float_to_bits(w[i * 4 + 1]), a0);
                    a1 = dot2_bf16(v[t][2], float_to_bits(w[i * 4 + 3]), a1);
                    acc[t][i][r][0] = a0;
                    acc[t][i][r][1] = a1;
                }
        }
    }
}

// NROWS rows of NW staged words each, row n at addr(n), handed to body(n, words) with the
// reads running one row ahead (PIPE, see k_rows_d2).
template <int NW, class Exec> NDC_D void read_row(Exec &ex, int at, uint32_t (&v)[NW])
{
    read_words<NW>(ex, at, v);
}

// `first`: row 0 already read by the caller (ahead of other work), or null.
template <int NROWS, int NW, bool PIPE, class Exec, class Addr, class Body>
NDC_D void stream_rows(Exec &ex, Addr addr, Body body, const uint32_t (*first)[NW] = nullptr)
{
    uint32_t vn[NW];
    if (PIPE) {
        if (first) {
            NDC_UNROLL
            for (int u = 0; u < NW; ++u) vn[u] = (*first)[u];
        } else {
            read_row<NW>(ex, addr(0), vn);
        }
    }
    NDC_UNROLL
    for (int n = 0; n < NROWS; ++n) {
        uint32_t v[NW];
        if (PIPE) {
            NDC_UNROLL
            for (int u = 0; u < NW; ++u) v[u] = vn[u];
            if (n + 1 < NROWS) read_words<NW>(ex, addr(n + 1), vn);
            ex.fence();
        } else {
            read_words<NW>(ex, addr(n), v);
        }
        body(n, v);
    }
}

// =================================================================== forward (bf16, dot2)

// KEEP: the call keeps s/d and n/d for backward (both tensors are there); without it the code
// that forms and stores them is not compiled in (as a run-time condition it cost a branch per
// row and channel, each reloading a spilled buffer resource).
template <int RH_, bool KEEP_ = false> struct FwdKernelB {
    static constexpr bool KEEP = KEEP_;
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    // staging slots per thread: thread (strip, lane) stages rows strip, strip + S, ... of the
    // TH + 4 source rows and TH + 2 x rows; with S >= kMinStrips strips, RH + 1 slots cover both
    static constexpr int kMinStrips = 4;
    static constexpr int RHK = RH + 1, NZR = RH + 1, NXR = RH + 1;
    // ring slots: source (one: it is only read in the scatter phase of the step that staged
    // it), x pairs, t1 pairs; plus one plane each of x and t1 as column-pair words (written
    // in the scatter phase, read in the gather phase of the same step)
    static constexpr int NS = 1, NX = 2, NTP = 2;
    static constexpr int kWavesPerSimd = 4;   // LDS leaves room for four workgroups per CU
    typedef bf16_t T;
    typedef FwdParams<T> Params;
    typedef VecIO<T, 2> IO;

    struct State {
        Lane ln;
        // BYTE offsets inside one plane (rows clamped; ooff: kNoAccess for a row outside the image)
        unsigned zoff[NZR], xoff[NXR], ooff[RH];
        unsigned zok, xok;
        float bv[SC];
        float t1acc[KD][RHK][RW];
        uint32_t t1prev[RHK];       // previous t1 plane of the own rows, as column pairs
        uint32_t pz[SC][NZR];       // staged source rows, raw (two bf16 columns per word)
        uint32_t px[NXR], pxprev[NXR];
    };

    static NDC_HD int rows_s(int TH) { return TH + 4; }
    static NDC_HD int rows_x(int TH) { return TH + 2; }
    // row pitch of a column-pair plane: W/2 words and a zero word on either side
    static NDC_HD int pitch_q(const Tile &t) { return t.CPW + 2; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        return (NS * 2 * rows_s(t.TH) + (NX + NTP) * rows_x(t.TH)) * t.P + 2 * rows_x(t.TH) * pitch_q(t);
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RS = rows_s(TH), RX = rows_x(TH);
        const int off_s = 0, off_x = NS * 2 * RS * P, off_t = off_x + NX * RX * P;
        const int PQ = pitch_q(t);
        const int off_qx = off_t + NTP * RX * P, off_qt = off_qx + RX * PQ;
        const int total = off_qt + RX * PQ;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        // this workgroup's (sample, channel) slices; offsets inside them fit 32 bits
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef xb_ = make_buf(p.x + cbase, xbytes), zb_ = make_buf(p.z + cbase * SC, sbytes);
        const BufRef ob_ = make_buf(p.out + cbase * SC, sbytes);
        const BufRef tb_ = make_buf(p.t1 ? p.t1 + cbase : nullptr, xbytes);
        const BufRef db_ = make_buf(KEEP ? p.s_over_den + cbase * SC : nullptr, sbytes);
        const BufRef rb_ = make_buf(KEEP ? p.ratio + cbase * SC : nullptr, sbytes);
        const bool have_t1 = p.t1 != nullptr;
        UniformF tab = as_uniform(p.wtab + (long long)id.c * kTabWords);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            if (k < D) {
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        st.pz[i][n] = buf_ld(zb_, st.zoff[n], (unsigned)k * plane2 + i * cplane2);
            }
            // planes outside the volume: load a clamped plane and select zero (a store in each
            // arm of a branch would push the staging registers into private memory)
            const int kx = k - PD;
            const bool xlive = kx >= 0 && kx < D;
            const unsigned xk = (unsigned)clampi(kx, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const uint32_t v = buf_ld(xb_, st.xoff[n], xk);
                st.px[n] = xlive ? v : 0u;
            }
        };

        // registers -> LDS: source plane k as channel-pair words into slot k % 3
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int lb = PL + st.ln.c0;
            const int sb = off_s + wrap(k % NS, NS) * 2 * RS * P;
            // planes past the end are never K-scattered, so their slot may keep stale words
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                if (k >= D || !((st.zok >> n) & 1u)) continue;
                const int j = st.ln.strip + n * S;
                float s[SC][RW];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    s[i][0] = bf_lo(st.pz[i][n]) + st.bv[i];
                    s[i][1] = bf_hi(st.pz[i][n]) + st.bv[i];
                    s[i][0] = floor_f(s[i][0], floor_);
                    s[i][1] = floor_f(s[i][1], floor_);
                }
                // the two columns of a channel pair one after the other: adjacent words, one
                // ds_write2_b32
                NDC_UNROLL
                for (int pr = 0; pr < 2; ++pr)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        ex.st_(sb + (pr * RS + j) * P + lb + c,
                               bits_to_float(pack_bf16x2(s[2 * pr][c], s[2 * pr + 1][c])));
            }
        };
        // x plane k - 1 completes the plane-pair word (x[k-2], x[k-1]) of slot (k - 2) % 2 and
        // is kept as column pairs for the gather of plane k - 2.
        // Runs in the scatter phase (a barrier after the gather that last read that slot), which
        // is what lets two slots do.
        auto store_x_pairs = [&](State &st, int k) NDC_LAMBDA {
            const int lb = PL + st.ln.c0;
            const int xb = off_x + wrap((k - 2) % NX, NX) * RX * P;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    const int j = st.ln.strip + n * S;
                    ex.st_(xb + j * P + lb, bits_to_float(zip_lo(st.pxprev[n], st.px[n])));
                    ex.st_(xb + j * P + lb + 1, bits_to_float(zip_hi(st.pxprev[n], st.px[n])));
                    // plane k - 1 as it came from memory: the column-pair word of this lane
                    ex.st_(off_qx + j * PQ + 1 + (st.ln.c0 >> 1), bits_to_float(st.px[n]));
                }
                st.pxprev[n] = st.px[n];
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.zok = st.xok = 0u;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RS && row >= 0 && row < H) st.zok |= 1u << n;
                st.zoff[n] = (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) st.pz[i][n] = 0u;
            }
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u;
                st.px[n] = st.pxprev[n] = 0u;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                st.ooff[r] = row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) st.bv[i] = p.bias ? p.bias[id.c * SC + i] : 0.f;
            NDC_UNROLL
            for (int r = 0; r < RHK; ++r) {
                st.t1prev[r] = 0u;
                NDC_UNROLL
                for (int c = 0; c < RW; ++c)
                    NDC_UNROLL
                    for (int a = 0; a < KD; ++a) st.t1acc[a][r][c] = 0.f;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();
        ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, 0); });
        ex.sync();

        // Two barriers per plane step: the source plane of the NEXT step is staged at the end of
        // the gather phase (nothing reads the source slot there), not in a phase of its own.
        for (int kk = 0; kk < D + 2; ++kk) {
            const int k = uniform_int(kk);   // the plane index stays on the scalar unit

            // ---- K-scatter of source plane k; t1 plane k - 1
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                store_x_pairs(st, k);
                const bool extra = st.ln.strip < 2;
                const int jx = halo_row(st.ln.strip, PH, TH);
                const int cb = PL + st.ln.c0 - PW;
                if (k < D) {
                    const int sb = off_s + wrap(k % NS, NS) * 2 * RS * P + cb;
                    NDC_ROLLED
                    for (int prr = 0; prr < 2; ++prr) {
                        const int pr = uniform_int(prr);
                        float wp[KT];
                        load_taps<KT>(tab + pr * KT, wp);
                        const int b0 = sb + pr * RS * P;
                        k_rows_d2<RH, RW, RHK, false>(ex, b0 + (PH + st.ln.strip * RH) * P, P, wp, st.t1acc, 0);
                        if (extra) k_rows_d2<1, RW, RHK, false>(ex, b0 + jx * P, P, wp, st.t1acc, RH);
                    }
                }
                // t1 plane k - 1 is complete: word (t1[k-2], t1[k-1]) goes to pair slot (k - 2) % 2
                const int pf = k - PD;
                const bool inplane = pf >= 0 && pf < D;
                const int tb = off_t + wrap((pf - 1) % NTP, NTP) * RX * P + PL + st.ln.c0;
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r) {
                    const bool mine = r < RH || extra;
                    const int j = r < RH ? PH + st.ln.strip * RH + r : jx;
                    const int row = r0 - PH + j;
                    const bool live = inplane && row >= 0 && row < H;
                    // the plane as column pairs: kept for the gather of plane k - 2, zipped with
                    // the previous plane's into the plane-pair words, and stored as t1
                    const uint32_t vq = live ? pack_bf16x2(st.t1acc[0][r][0], st.t1acc[0][r][1]) : 0u;
                    if (mine) {
                        ex.st_(tb + j * P, bits_to_float(zip_lo(st.t1prev[r], vq)));
                        ex.st_(tb + j * P + 1, bits_to_float(zip_hi(st.t1prev[r], vq)));
                        ex.st_(off_qt + j * PQ + 1 + (st.ln.c0 >> 1), bits_to_float(vq));
                    }
                    st.t1prev[r] = vq;
                    if (r < RH && have_t1 && live)
                        buf_st(tb_, st.ooff[r < RH ? r : 0], (unsigned)pf * plane2, vq);
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        st.t1acc[0][r][c] = st.t1acc[1][r][c];
                        st.t1acc[1][r][c] = st.t1acc[2][r][c];
                        st.t1acc[2][r][c] = 0.f;
                    }
                }
            });
            ex.sync();

            // ---- prefetch, then A-gather + epilogue of plane k - 2, then staging of plane k + 1
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                load_plane(st, k + 1);
                const int j0 = k - 2;
                if (j0 < 0) {
                    store_plane(st, k + 1);
                    return;
                }
                // the thread's own source values of plane j0: z is read again (it was staged two
                // steps ago, so this hits the L2) rather than kept in LDS or registers that long
                uint32_t own[SC][RH];
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        own[i][r] = buf_ld(zb_, st.ooff[r], (unsigned)j0 * plane2 + i * cplane2);
                float acc[2][SC][RH][RW];   // n, d: their sums start at eps (first pass below)
                {
                    // depth taps 2 and 1 from the plane-pair words (x, t1)[j0-1 .. j0]
                    float wt[SC][9];
                    load_plane_taps<SC, 9, 9>(tab + kTabWA, wt);
                    const int m = j0 - 1;
                    const int ob = (st.ln.strip * RH) * P + PL + st.ln.c0 - PW;
                    const int base[2] = {off_x + wrap(m % NX, NX) * RX * P + ob,
                                         off_t + wrap(m % NTP, NTP) * RX * P + ob};
                    a_plane_d2<RH, RW, 2, false, true>(ex, base, P, wt, acc, eps);
                }
                {
                    // depth tap 0 from the column-pair words of plane j0 + 1
                    const int oq = (st.ln.strip * RH) * PQ + (st.ln.c0 >> 1);
                    const int base[2] = {off_qx + oq, off_qt + oq};
                    a_plane_q<RH, 2>(ex, base, PQ, tab + kTabWQ, acc);
                }
                const unsigned oj = (unsigned)j0 * plane2;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    // (a row outside the image: its stores go nowhere)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v[RW], rd[RW], rt[RW];
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            const uint32_t w = own[i][r];
                            // same arithmetic as the staging, so s is the staged value before
                            // its rounding to bf16
                            const float s = floor_f((c ? bf_hi(w) : bf_lo(w)) + st.bv[i], floor_);
                            const float inv = fast_rcp(acc[1][i][r][c]);
                            rd[c] = s * inv;
                            rt[c] = acc[0][i][r][c] * inv;
                            v[c] = s * rt[c];
                        }
                        buf_st<true>(ob_, st.ooff[r], oj + i * cplane2, pack_bf16x2(v[0], v[1]));
                        if (KEEP) {
                            buf_st<true>(db_, st.ooff[r], oj + i * cplane2, pack_bf16x2(rd[0], rd[1]));
                            buf_st<true>(rb_, st.ooff[r], oj + i * cplane2, pack_bf16x2(rt[0], rt[1]));
                        }
                    }
                }
                store_plane(st, k + 1);
            });
            ex.sync();
        }
    }
};

// =================================================================== backward pass 1 (bf16, dot2)

// SAVED: the call brings the forward's s/d and n/d, so gn = g (s/d), gd = -gn (n/d) are
// elementwise (z is not read) and the plane-pair rings of x and t1 (for re-gathering n and d)
// are not kept.
template <int RH_, bool SAVED_ = false> struct Bwd1KernelB {
    static constexpr bool SAVED = SAVED_;
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int NXR = RH + 2;
    static constexpr int NP = 2, NXT = 3;   // ring slots: plane pairs of x / t1; (x, t1) words
    static constexpr int NRED = SC * KT;
    typedef bf16_t T;
    typedef BwdParams<T> Params;

    struct State {
        Lane ln;
        // byte offsets inside one plane; ooff / hoff: kNoAccess for a row outside the image
        unsigned xoff[NXR], ooff[RH];
        unsigned xok;
        float bv[SC];
        float gacc[SC][KT];
        float accx[KD][RH][RW], acct[KD][RH][RW];
        uint32_t px[NXR], pt[NXR], pxprev[NXR], ptprev[NXR];
        // SAVED: gout, s/d, n/d words of the next plane, fetched one phase ahead (own rows,
        // then the halo row of the first two strips)
        uint32_t qg[SC][RH + 1], qd[SC][RH + 1], qr[SC][RH + 1];
        unsigned hoff;
        // LDS word offsets inside a ring slot, formed once: the word (first own row - 1, first
        // own column - 1) of an (x, t1) slot's rows, the word (row `strip`, first own column),
        // and the word (halo row, first own column) of a gn/gd plane.  What is added per access
        // (slot, row) is the same in every lane and stays on the scalar unit.
        int ob, so, ho;
    };

    static NDC_HD int rows_x(int TH) { return TH + 4; }
    static NDC_HD int rows_g(int TH) { return TH + 2; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = (((SAVED ? 0 : 2 * NP) + NXT) * rows_x(t.TH) + 4 * rows_g(t.TH)) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH), RG = rows_g(TH);
        const int SP = S * P;
        const int off_xp = 0, off_tp = NP * RX * P, off_xt = SAVED ? 0 : 2 * NP * RX * P;
        const int off_g = off_xt + NXT * RX * P;
        const int total = off_g + 4 * RG * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        // this workgroup's (sample, channel) slices; offsets inside them fit 32 bits
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef xb_ = make_buf(p.x + cbase, xbytes), tb_ = make_buf(p.t1 + cbase, xbytes);
        const BufRef zb_ = make_buf(SAVED ? nullptr : p.z + cbase * SC, sbytes);
        const BufRef gb_ = make_buf(p.gout + cbase * SC, sbytes);
        const BufRef db_ = make_buf(SAVED ? p.s_over_den + cbase * SC : nullptr, sbytes);
        const BufRef rb_ = make_buf(SAVED ? p.ratio + cbase * SC : nullptr, sbytes);
        const BufRef gxb_ = make_buf(p.gx ? p.gx + cbase : nullptr, xbytes);
        const BufRef gtb_ = make_buf(p.gt1 + cbase, xbytes);
        const bool have_gx = p.gx != nullptr;
        UniformF tab = as_uniform(p.wtab + (long long)id.c * kTabWords);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;
        const int need_gh = p.need_gh;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            // (every lane issues every fetch, lanes outside the tile with offsets outside the
            // slices: a fetch under a condition gives the compiler a path without it, on which
            // it cannot count the outstanding loads and makes every user wait for all of them)
            // planes past the end: load the last plane and select zero (a store in each arm of
            // a branch would push the staging registers into private memory)
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const uint32_t vx = buf_ld(xb_, st.xoff[n], ko);
                const uint32_t vt = buf_ld(tb_, st.xoff[n], ko);
                st.px[n] = live ? vx : 0u;
                st.pt[n] = live ? vt : 0u;
            }
        };
        // plane k arrives: plane-pair words (v[k-1], v[k]) into pair slot (k-1) % 2 and the
        // operand-pair words (x[k], t1[k]) into slot k % 3
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int ps = wrap((k - 1) % NP, NP) * RX * P, xs = wrap(k % NXT, NXT) * RX * P;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    const int o = st.so + n * SP;
                    if (!SAVED) {
                        ex.st_(off_xp + ps + o, bits_to_float(zip_lo(st.pxprev[n], st.px[n])));
                        ex.st_(off_xp + ps + o + 1, bits_to_float(zip_hi(st.pxprev[n], st.px[n])));
                        ex.st_(off_tp + ps + o, bits_to_float(zip_lo(st.ptprev[n], st.pt[n])));
                        ex.st_(off_tp + ps + o + 1, bits_to_float(zip_hi(st.ptprev[n], st.pt[n])));
                    }
                    ex.st_(off_xt + xs + o, bits_to_float(zip_lo(st.px[n], st.pt[n])));
                    ex.st_(off_xt + xs + o + 1, bits_to_float(zip_hi(st.px[n], st.pt[n])));
                }
                st.pxprev[n] = st.px[n];
                st.ptprev[n] = st.pt[n];
            }
        };

        // gn, gd of NR rows from gn/gd tile row j (image row r0 - 1 + j): published to LDS as
        // channel-pair words; returned as operand pairs GG[i][r][c] = (gn_i, gd_i)
        // SAVED: fetch plane jn of gout, s/d, n/d into the state, a phase before it is used
        auto prefetch_g = [&](State &st, int jn) NDC_LAMBDA {
            if (!SAVED) return;
            // (past the last plane a clamped plane is fetched and never used: no branch
            // around loads, see load_plane)
            const unsigned jo = (unsigned)clampi(jn, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int r = 0; r < RH + 1; ++r) {
                if (r == RH && st.ln.strip >= 2) continue;
                const unsigned o = r < RH ? st.ooff[r < RH ? r : 0] : st.hoff;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    st.qg[i][r] = buf_ld<true>(gb_, o, jo + i * cplane2);
                    st.qd[i][r] = buf_ld<true>(db_, o, jo + i * cplane2);
                    st.qr[i][r] = buf_ld<true>(rb_, o, jo + i * cplane2);
                }
            }
        };

        // roff: where the rows sit in the prefetched words (0: own rows, RH: halo row)
        // lo: LDS word offset of (tile row j, first own column) inside a plane
        auto gn_gd_rows = [&](State &st, int j1, int j, int lo, auto nr_tag, int roff,
                              uint32_t (&gg_out)[SC][decltype(nr_tag)::value][RW]) NDC_LAMBDA {
            constexpr int NR = decltype(nr_tag)::value;
            uint32_t zw[SC][NR], gw[SC][NR], dw[SC][NR], rw[SC][NR];
            const unsigned jo = (unsigned)j1 * plane2;
            bool ok[NR];
            NDC_UNROLL
            for (int r = 0; r < NR; ++r) {
                const int row = r0 - PH + j + r;
                ok[r] = row >= 0 && row < H;
                const unsigned o = (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    if (SAVED) {
                        zw[i][r] = 0u;
                        gw[i][r] = st.qg[i][roff + r];
                        dw[i][r] = st.qd[i][roff + r];
                        rw[i][r] = st.qr[i][roff + r];
                    } else {
                        gw[i][r] = buf_ld(gb_, o, jo + i * cplane2);
                        zw[i][r] = buf_ld(zb_, o, jo + i * cplane2);
                        dw[i][r] = rw[i][r] = 0u;
                    }
                }
            }
            float acc[2][SC][NR][RW];
            NDC_UNROLL
            for (int a = 0; a < 2; ++a)
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int r = 0; r < NR; ++r)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) acc[a][i][r][c] = eps;
            if (!SAVED) {
                NDC_ROLLED
                for (int s = 0; s < 2; ++s) {
                    float wt[SC][9];
                    load_plane_taps<SC, 9, 9>(tab + 54 + s * 36, wt);
                    const int m = j1 - 1 + s;
                    const int ob = lo - PW + wrap(m % NP, NP) * RX * P;
                    const int base[2] = {off_xp + ob, off_tp + ob};
                    a_plane_d2<NR, RW, 2, true>(ex, base, P, wt, acc);
                }
            }
            NDC_UNROLL
            for (int r = 0; r < NR; ++r) {
                float gn[SC][RW], gd[SC][RW];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        const float sv = floor_f((c ? bf_hi(zw[i][r]) : bf_lo(zw[i][r])) + st.bv[i], floor_);
                        // SAVED: the words of a row outside the image were read as zeros
                        const float g_ = c ? bf_hi(gw[i][r]) : bf_lo(gw[i][r]);
                        const float gv = SAVED || ok[r] ? g_ : 0.f;
                        if (SAVED) {
                            gn[i][c] = gv * (c ? bf_hi(dw[i][r]) : bf_lo(dw[i][r]));
                            gd[i][c] = -(gn[i][c] * (c ? bf_hi(rw[i][r]) : bf_lo(rw[i][r])));
                        } else {
                            const float inv = fast_rcp(acc[1][i][r][c]);
                            gn[i][c] = gv * sv * inv;
                            gd[i][c] = -(gn[i][c] * acc[0][i][r][c]) * inv;
                        }
                        gg_out[i][r][c] = pack_bf16x2(gn[i][c], gd[i][c]);
                    }
                // (the two columns of each word plane one after the other: adjacent words, one
                // ds_write2_b32)
                const int o = lo + (off_g + r * P);
                NDC_UNROLL
                for (int pr = 0; pr < 2; ++pr)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        ex.st_(o + pr * RG * P + c, bits_to_float(pack_bf16x2(gn[2 * pr][c], gn[2 * pr + 1][c])));
                NDC_UNROLL
                for (int pr = 0; pr < 2; ++pr)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        ex.st_(o + (2 + pr) * RG * P + c, bits_to_float(pack_bf16x2(gd[2 * pr][c], gd[2 * pr + 1][c])));
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.xok = 0u;
            st.ob = st.ln.strip * RH * P + PL + st.ln.c0 - PW;
            st.so = st.ln.strip * P + PL + st.ln.c0;
            st.ho = halo_row(st.ln.strip, PH, TH) * P + PL + st.ln.c0;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = st.ln.active ? (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u : kNoAccess;
                st.px[n] = st.pt[n] = st.pxprev[n] = st.ptprev[n] = 0u;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                st.ooff[r] = st.ln.active && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
            }
            {
                const int hrow = r0 - PH + halo_row(st.ln.strip, PH, TH);
                st.hoff = st.ln.active && hrow >= 0 && hrow < H ? (unsigned)(hrow * W + st.ln.c0) * 2u : kNoAccess;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int r = 0; r < RH + 1; ++r) st.qg[i][r] = st.qd[i][r] = st.qr[i][r] = 0u;
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
            load_plane(st, 0);
        });
        ex.sync();
        ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, 0); });
        ex.sync();

        // Two barriers per plane step: the (x, t1) plane of the NEXT step is staged at the end
        // of the scatter phase (the ring slots it overwrites were last read in the phase before).
        for (int kk = 0; kk < D + 2; ++kk) {
            const int k = uniform_int(kk);   // the plane index stays on the scalar unit

            const int j1 = k - 1;
            const bool live1 = j1 >= 0 && j1 < D;
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active || !live1) return;
                {
                    uint32_t gg2[SC][RH][RW];
                    const int j = PH + st.ln.strip * RH;
                    auto xt_row = [&](int n) NDC_LAMBDA {
                        const int td = n / (RH + 2), q = n % (RH + 2);
                        return st.ob + (off_xt + (wrap((j1 + 1 - td) % NXT, NXT) * RX + PH + q) * P);
                    };
                    // the first (x, t1) row of the filter-gradient stream is requested before
                    // the elementwise work, so that it has arrived when that is done
                    uint32_t row0[RW + 2];
                    read_row<RW + 2>(ex, xt_row(0), row0);
                    ex.fence();
                    gn_gd_rows(st, j1, j, st.ob + (PW + PH * P), IntTag<RH>(), 0, gg2);
                    if (need_gh) {
                        // A-side filter-gradient terms: (gn_i, gd_i) . (x, t1)[neighbour]
                        stream_rows<KD * (RH + 2), RW + 2, true>(
                            ex, xt_row,
                            [&](int n, const uint32_t (&v)[RW + 2]) NDC_LAMBDA {
                                const int td = n / (RH + 2), q = n % (RH + 2);
                                NDC_UNROLL
                                for (int th = 0; th < KH; ++th) {
                                    const int rr = q - 2 + th;
                                    if (rr >= 0 && rr < RH) {
                                        NDC_UNROLL
                                        for (int tw = 0; tw < KW; ++tw)
                                            NDC_UNROLL
                                            for (int i = 0; i < SC; ++i)
                                                NDC_UNROLL
                                                for (int c = 0; c < RW; ++c)
                                                    st.gacc[i][(td * KH + th) * KW + tw] = dot2_bf16(
                                                        v[c + 2 - tw], gg2[i][rr][c],
                                                        st.gacc[i][(td * KH + th) * KW + tw]);
                                    }
                                }
                            }, &row0);
                    }
                }
                if (st.ln.strip < 2) {
                    uint32_t gg1[SC][1][RW];
                    gn_gd_rows(st, j1, halo_row(st.ln.strip, PH, TH), st.ho, IntTag<1>(), RH, gg1);
                }
            });
            ex.sync();

            ex.each([&](State &st, int) NDC_LAMBDA {
                load_plane(st, k + 1);
                prefetch_g(st, k);
                if (!st.ln.active) return;
                if (live1) {
                    const int gb_ = st.ob + off_g;
                    // the two channel pairs one after the other in straight-line code (as a
                    // rolled loop the accumulators it carries were permuted by register copies
                    // on every trip); the fence keeps the second pair's tap loads behind the
                    // first pair's arithmetic
                    NDC_UNROLL
                    for (int pr = 0; pr < 2; ++pr) {
                        ex.fence();
                        float wp[KT];
                        load_taps<KT>(tab + pr * KT, wp);
                        // gn rows of this channel pair feed gx, then its gd rows feed gt1
                        stream_rows<2 * (RH + 2), RW + 2, true>(
                            ex,
                            [&](int n) NDC_LAMBDA {
                                return gb_ + ((n / (RH + 2)) * 2 + pr) * RG * P + (n % (RH + 2)) * P;
                            },
                            [&](int n, const uint32_t (&v)[RW + 2]) NDC_LAMBDA {
                                if (n < RH + 2)
                                    k_row_d2<RH, RW, RH>(n, v, wp, st.accx, 0);
                                else
                                    k_row_d2<RH, RW, RH>(n - (RH + 2), v, wp, st.acct, 0);
                            });
                    }
                }
                const int pf = k - 2;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (pf >= 0) {   // rows outside the image: the stores go nowhere
                        if (have_gx) buf_st<true>(gxb_, st.ooff[r], (unsigned)pf * plane2,
                                            pack_bf16x2(st.accx[0][r][0], st.accx[0][r][1]));
                        buf_st(gtb_, st.ooff[r], (unsigned)pf * plane2,
                               pack_bf16x2(st.acct[0][r][0], st.acct[0][r][1]));
                    }
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        st.accx[0][r][c] = st.accx[1][r][c];
                        st.accx[1][r][c] = st.accx[2][r][c];
                        st.accx[2][r][c] = 0.f;
                        st.acct[0][r][c] = st.acct[1][r][c];
                        st.acct[1][r][c] = st.acct[2][r][c];
                        st.acct[2][r][c] = 0.f;
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

// =================================================================== backward pass 2 (bf16, dot2)

// SAVED: gz = [s > 0] (g (n/d) + A(gt1)) with the forward's n/d, so only the gt1 ring is kept.
template <int RH_, bool SAVED_ = false> struct Bwd2KernelB {
    static constexpr bool SAVED = SAVED_;
    static constexpr int NA = SAVED ? 1 : 3;   // gathered operands: (x, t1,) gt1
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int NXR = RH + 1;
    static constexpr int NP = 3, NG = 4;   // ring slots: plane pairs of x / t1; of gt1
    static constexpr int NRED = SC * KT + SC;
    typedef bf16_t T;
    typedef BwdParams<T> Params;

    struct State {
        Lane ln;
        unsigned xoff[NXR], ooff[RH];
        unsigned xok;
        // bias per own row: the channel's bias; for a row outside the image (whose z, gout,
        // n/d words read as zeros) -1 when the source is rectified and 0 when it is not, so
        // that its source values and rectified gradients come out as zeros without a select
        float bvr[SC][RH];
        // (1, 1) as a bf16 pair for a row inside the image, (0, 0) outside: the weights of the
        // row's gz words in gb (gb sums the gz values as they are stored, one dot2 per word)
        uint32_t okw[RH];
        float gacc[SC][KT];
        float gbacc[SC];
        float sprev[SC][RH][RW];   // own source values of the previous plane
        uint32_t px[NXR], pt[NXR], pg[NXR], pxprev[NXR], ptprev[NXR], pgprev[NXR];
        // SAVED: the z, gout, n/d words of two planes: the step of plane parity P works on set P
        // and fetches the next plane's into set 1 - P (the plane loop is unrolled twice, so
        // the sets are fixed registers and nothing is copied from step to step)
        uint32_t qz[2][SC][RH], qg[2][SC][RH], qr[2][SC][RH];
        // LDS word offsets inside a ring slot, formed once: the word (first own row - 1, first
        // own column - 1) and the word (row `strip`, first own column).  What is added per
        // access (slot, row) is the same in every lane and stays on the scalar unit.
        int ob, so;
    };

    static NDC_HD int rows_x(int TH) { return TH + 2; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int main_ = ((SAVED ? 0 : 2 * NP) + NG) * rows_x(t.TH) * t.P;
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RX = rows_x(TH);
        const int SP = S * P;
        const int off_xp = 0, off_tp = NP * RX * P, off_gp = SAVED ? 0 : 2 * NP * RX * P;
        const int total = off_gp + NG * RX * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        // this workgroup's (sample, channel) slices; offsets inside them fit 32 bits
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef xb_ = make_buf(SAVED ? nullptr : p.x + cbase, xbytes);
        const BufRef tb_ = make_buf(SAVED ? nullptr : p.t1 + cbase, xbytes);
        const BufRef gtb_ = make_buf(p.gt1 + cbase, xbytes);
        const BufRef zb_ = make_buf(p.z + cbase * SC, sbytes), gb_ = make_buf(p.gout + cbase * SC, sbytes);
        const BufRef rb_ = make_buf(SAVED ? p.ratio + cbase * SC : nullptr, sbytes);
        const BufRef gzb_ = make_buf(p.gz ? p.gz + cbase * SC : nullptr, sbytes);
        UniformF tab = as_uniform(p.wtab + (long long)id.c * kTabWords);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();   // floor_f(s, floor_) rectifies or passes through
        const float eps = p.eps;
        const int need_gh = p.need_gh;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            // (every lane issues every fetch, lanes outside the tile with offsets outside the
            // slices: a fetch under a condition gives the compiler a path without it, on which
            // it cannot count the outstanding loads and makes every user wait for all of them)
            // planes past the end: load the last plane and select zero (a store in each arm of
            // a branch would push the staging registers into private memory)
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const uint32_t vx = SAVED ? 0u : buf_ld(xb_, st.xoff[n], ko);
                const uint32_t vt = SAVED ? 0u : buf_ld(tb_, st.xoff[n], ko);
                const uint32_t vg = buf_ld(gtb_, st.xoff[n], ko);
                st.px[n] = live ? vx : 0u;
                st.pt[n] = live ? vt : 0u;
                st.pg[n] = live ? vg : 0u;
            }
        };
        // plane k arrives: plane-pair words (v[k-1], v[k]) into slot (k-1) % ring
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int ps = wrap((k - 1) % NP, NP) * RX * P, gs = wrap((k - 1) % NG, NG) * RX * P;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    const int o = st.so + n * SP;
                    if (!SAVED) {
                        ex.st_(off_xp + ps + o, bits_to_float(zip_lo(st.pxprev[n], st.px[n])));
                        ex.st_(off_xp + ps + o + 1, bits_to_float(zip_hi(st.pxprev[n], st.px[n])));
                        ex.st_(off_tp + ps + o, bits_to_float(zip_lo(st.ptprev[n], st.pt[n])));
                        ex.st_(off_tp + ps + o + 1, bits_to_float(zip_hi(st.ptprev[n], st.pt[n])));
                    }
                    ex.st_(off_gp + gs + o, bits_to_float(zip_lo(st.pgprev[n], st.pg[n])));
                    ex.st_(off_gp + gs + o + 1, bits_to_float(zip_hi(st.pgprev[n], st.pg[n])));
                }
                st.pxprev[n] = st.px[n];
                st.ptprev[n] = st.pt[n];
                st.pgprev[n] = st.pg[n];
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.xok = 0u;
            st.ob = st.ln.strip * RH * P + PL + st.ln.c0 - PW;
            st.so = st.ln.strip * P + PL + st.ln.c0;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = st.ln.active ? (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u : kNoAccess;
                st.px[n] = st.pt[n] = st.pg[n] = st.pxprev[n] = st.ptprev[n] = st.pgprev[n] = 0u;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                // a row outside the image: its loads give 0 and its stores go nowhere
                st.ooff[r] = st.ln.active && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
                st.okw[r] = row < H ? 0x3f803f80u : 0u;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    st.bvr[i][r] = row < H ? (p.bias ? p.bias[id.c * SC + i] : 0.f) : (p.relu ? -1.f : 0.f);
            }
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) {
                st.gbacc[i] = 0.f;
                NDC_UNROLL
                for (int a = 0; a < KT; ++a) st.gacc[i][a] = 0.f;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) st.sprev[i][r][c] = 0.f;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    NDC_UNROLL
                    for (int a = 0; a < 2; ++a) st.qz[a][i][r] = st.qg[a][i][r] = st.qr[a][i][r] = 0u;
            }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        // one step past the usual end so that an unpaired last plane still gets its
        // filter-gradient contribution (paired with a zero plane)
        // one plane step; PAR = k % 2, known at compile time (the loop below is unrolled twice)
        auto compute = [&](State &st, int k, auto par_tag) NDC_LAMBDA {
                constexpr int PAR = decltype(par_tag)::value;
                const int j0 = k - 1;
                load_plane(st, k + 1);
                // SAVED: this plane's z, gout, n/d words were fetched a step ago; take them and
                // start the fetch of the next plane's
                uint32_t zw[SC][RH], gw[SC][RH], rw[SC][RH];
                if (SAVED) {
                    const unsigned jn = (unsigned)clampi(k, 0, D - 1) * plane2;
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int i = 0; i < SC; ++i) {
                            zw[i][r] = st.qz[PAR][i][r];
                            gw[i][r] = st.qg[PAR][i][r];
                            rw[i][r] = st.qr[PAR][i][r];
                            st.qz[1 - PAR][i][r] = buf_ld(zb_, st.ooff[r], jn + i * cplane2);
                            st.qg[1 - PAR][i][r] = buf_ld<true>(gb_, st.ooff[r], jn + i * cplane2);
                            st.qr[1 - PAR][i][r] = buf_ld<true>(rb_, st.ooff[r], jn + i * cplane2);
                        }
                }
                if (!st.ln.active || j0 < 0) return;
                float sv[SC][RH][RW];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) sv[i][r][c] = 0.f;
                if (j0 < D) {
                    const unsigned jo = (unsigned)j0 * plane2;
                    if (!SAVED) {
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int i = 0; i < SC; ++i) {
                                zw[i][r] = buf_ld(zb_, st.ooff[r], jo + i * cplane2);
                                gw[i][r] = buf_ld(gb_, st.ooff[r], jo + i * cplane2);
                                rw[i][r] = 0u;
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
                                for (int c = 0; c < RW; ++c) {
                                    // SAVED: the sum starts from g (n/d), the other term of gz
                                    if (SAVED)
                                        acc[a][i][r][c] = (c ? bf_hi(gw[i][r]) : bf_lo(gw[i][r])) *
                                                          (c ? bf_hi(rw[i][r]) : bf_lo(rw[i][r]));
                                    else
                                        acc[a][i][r][c] = a < NA - 1 ? eps : 0.f;
                                }
                    NDC_ROLLED
                    for (int s = 0; s < 2; ++s) {
                        float wt[SC][9];
                        load_plane_taps<SC, 9, 9>(tab + 54 + s * 36, wt);
                        const int m = j0 - 1 + s;
                        int base[NA];
                        base[NA - 1] = st.ob + (off_gp + wrap(m % NG, NG) * RX * P);
                        if (!SAVED) {
                            base[0] = st.ob + (off_xp + wrap(m % NP, NP) * RX * P);
                            base[NA > 1 ? 1 : 0] = st.ob + (off_tp + wrap(m % NP, NP) * RX * P);
                        }
                        a_plane_d2<RH, RW, NA, SAVED>(ex, base, P, wt, acc);
                    }
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r) {
                        NDC_UNROLL
                        for (int i = 0; i < SC; ++i) {
                            float v[RW];
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) {
                                const float s = floor_f((c ? bf_hi(zw[i][r]) : bf_lo(zw[i][r])) + st.bvr[i][r], floor_);
                                float gzv;
                                if (SAVED)
                                    gzv = acc[NA - 1][i][r][c];
                                else
                                    gzv = (c ? bf_hi(gw[i][r]) : bf_lo(gw[i][r])) * acc[0][i][r][c] *
                                              fast_rcp(acc[NA > 1 ? 1 : 0][i][r][c]) +
                                          acc[NA - 1][i][r][c];
                                if (p.relu && s <= 0.f) gzv = 0.f;   // a NaN passes
                                sv[i][r][c] = s;
                                v[c] = gzv;
                            }
                            const uint32_t gzw = pack_bf16x2(v[0], v[1]);
                            st.gbacc[i] = dot2_bf16(gzw, st.okw[r], st.gbacc[i]);
                            // (no gz asked for: gzb_ is an empty slice and the store goes nowhere)
                            buf_st<true>(gzb_, st.ooff[r], jo + i * cplane2, gzw);
                        }
                    }
                }
                if (PAR == 0 && need_gh && j0 <= D) {   // j0 odd
                    // K-side filter-gradient term for the plane pair (j0 - 1, j0):
                    // (s_i[j0-1], s_i[j0]) . (gt1[m], gt1[m+1])[neighbour], m = j0 - td
                    uint32_t ss[SC][RH][RW];
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) ss[i][r][c] = pack_bf16x2(st.sprev[i][r][c], sv[i][r][c]);
                    stream_rows<KD * (RH + 2), RW + 2, SAVED>(
                        ex,
                        [&](int n) NDC_LAMBDA {
                            const int td = n / (RH + 2), q = n % (RH + 2);
                            return st.ob + (off_gp + (wrap((j0 - td) % NG, NG) * RX + q) * P);
                        },
                        [&](int n, const uint32_t (&v)[RW + 2]) NDC_LAMBDA {
                            const int td = n / (RH + 2), q = n % (RH + 2);
                            NDC_UNROLL
                            for (int th = 0; th < KH; ++th) {
                                const int rr = q - 2 + th;
                                if (rr >= 0 && rr < RH) {
                                    NDC_UNROLL
                                    for (int tw = 0; tw < KW; ++tw)
                                        NDC_UNROLL
                                        for (int i = 0; i < SC; ++i)
                                            NDC_UNROLL
                                            for (int c = 0; c < RW; ++c)
                                                st.gacc[i][(td * KH + th) * KW + tw] = dot2_bf16(
                                                    v[c + 2 - tw], ss[i][rr][c],
                                                    st.gacc[i][(td * KH + th) * KW + tw]);
                                }
                            }
                        });
                }
                if (PAR == 1) {   // j0 even: the next step pairs this plane's source values with its own
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) st.sprev[i][r][c] = sv[i][r][c];
                }
        };
        for (int kk = 0; kk < D + 2; kk += 2) {
            {
                const int k = uniform_int(kk);   // the plane index stays on the scalar unit
                ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k); });
                ex.sync();
                ex.each([&](State &st, int) NDC_LAMBDA { compute(st, k, IntTag<0>()); });
            }
            {   // (always: an even number of steps, the last possibly past the end of the march,
                // where it finds nothing to do; under a condition the compiler sees a path
                // from one even step to the next without this step's loads and can no longer
                // count the loads outstanding)
                const int k = uniform_int(kk + 1);
                ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k); });
                ex.sync();
                ex.each([&](State &st, int) NDC_LAMBDA { compute(st, k, IntTag<1>()); });
            }
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
