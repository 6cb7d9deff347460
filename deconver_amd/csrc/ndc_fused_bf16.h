// bfloat16 variants of the fused kernels for the 3x3x3, SC = 4 depthwise geometry, built on
// v_dot2c_f32_bf16 (two bf16 MACs per lane-instruction, float32 accumulate, same issue
// rate as an fp32 FMA).  Same work decomposition, rings and march as ndc_fused.h; what
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
#pragma once

#include "ndc_fused.h"

namespace ndc {
namespace fused {

static const int kTabWords = 126;   // packed tap words per channel (54 WK + 72 WA)

// idx over C * kTabWords
NDC_HD void prep_tables(long long idx, const float *h, float *tab)
{
    const int c = (int)(idx / kTabWords), e = (int)(idx % kTabWords);
    const float *hc = h + (long long)c * 4 * 27;
    uint32_t w;
    if (e < 54) {
        const int p = e / 27, tau = e % 27;
        w = pack_bf16x2(hc[(2 * p) * 27 + tau], hc[(2 * p + 1) * 27 + tau]);
    } else {
        const int r = e - 54, s = r / 36, i = (r % 36) / 9, t9 = r % 9;
        w = s == 0 ? pack_bf16x2(hc[i * 27 + 2 * 9 + t9], hc[i * 27 + 1 * 9 + t9])
                   : pack_bf16x2(0.f, hc[i * 27 + t9]);
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

// K-type pass over an NR x RW tile for ONE channel pair: words (s_2p, s_2p+1) staged at
// `base` (first input row, first own column - 1); w = WK[p], 27 packed tap pairs.
template <int NR, int RW, int STRIDE, class Exec>
NDC_D void k_rows_d2(Exec &ex, int base, int P, const float (&w)[27], float (*acc)[STRIDE][RW],
                     int r_off)
{
    NDC_UNROLL
    for (int q = 0; q < NR + 2; ++q) {
        uint32_t v[RW + 2];
        NDC_UNROLL
        for (int u = 0; u < RW + 2; ++u) v[u] = float_to_bits(ex.ld(base + q * P + u));
        NDC_UNROLL
        for (int th = 0; th < 3; ++th) {
            const int rr = q - th;
            if (rr < 0 || rr >= NR) continue;
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

// A-type pass over an NR x RW tile for one plane-pair slot of NTEN operands; wt = WA[s].
template <int NR, int RW, int NTEN, class Exec>
NDC_D void a_plane_d2(Exec &ex, const int (&base)[NTEN], int P, const float (&wt)[4][9],
                      float (&acc)[NTEN][4][NR][RW])
{
    NDC_UNROLL
    for (int q = 0; q < NR + 2; ++q) {
        uint32_t v[NTEN][RW + 2];
        NDC_UNROLL
        for (int t = 0; t < NTEN; ++t)
            NDC_UNROLL
            for (int u = 0; u < RW + 2; ++u) v[t][u] = float_to_bits(ex.ld(base[t] + q * P + u));
        NDC_UNROLL
        for (int th = 0; th < 3; ++th) {
            const int rr = q - 2 + th;
            if (rr < 0 || rr >= NR) continue;
            NDC_UNROLL
            for (int tw = 0; tw < 3; ++tw)
                NDC_UNROLL
                for (int i = 0; i < 4; ++i) {
                    const uint32_t wv = float_to_bits(wt[i][th * 3 + tw]);
                    NDC_UNROLL
                    for (int t = 0; t < NTEN; ++t)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c)
                            acc[t][i][rr][c] = dot2_bf16(v[t][c + 2 - tw], wv, acc[t][i][rr][c]);
                }
        }
    }
}

// =================================================================== forward (bf16, dot2)

template <int RH_> struct FwdKernelB {
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int RHK = RH + 1, NZR = RH + 2, NXR = RH + 1;
    static constexpr int NS = 3, NX = 3, NTP = 2;   // ring slots: source, x pairs, t1 pairs
    typedef bf16_t T;
    typedef FwdParams<T> Params;
    typedef VecIO<T, 2> IO;

    struct State {
        Lane ln;
        int zoff[NZR], xoff[NXR], ooff[RH];
        unsigned zok, xok, ook;
        float bv[SC];
        float t1acc[KD][RHK][RW];
        float t1prev[RHK][RW];
        uint32_t pz[SC][NZR];       // staged source rows, raw (two bf16 columns per word)
        uint32_t px[NXR], pxprev[NXR];
        uint32_t own[2][RH][RW];    // the thread's own source words of the plane being finished
    };

    static NDC_HD int rows_s(int TH) { return TH + 4; }
    static NDC_HD int rows_x(int TH) { return TH + 2; }
    static NDC_HD int lds_floats(const Tile &t)
    {
        return (NS * 2 * rows_s(t.TH) + (NX + NTP) * rows_x(t.TH)) * t.P;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t);
        const int S = t.S, P = t.P, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int RS = rows_s(TH), RX = rows_x(TH);
        const int off_s = 0, off_x = NS * 2 * RS * P, off_t = off_x + NX * RX * P;
        const int total = off_t + NTP * RX * P;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const T *xg = p.x + ((long long)id.b * p.C + id.c) * cplane;
        const T *zg = p.z + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *og = p.out + ((long long)id.b * p.C + id.c) * SC * cplane;
        T *t1g = p.t1 ? p.t1 + ((long long)id.b * p.C + id.c) * cplane : nullptr;
        UniformF tab = as_uniform(p.wtab + (long long)id.c * kTabWords);
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const int relu = p.relu;
        const float eps = p.eps;

        auto load_plane = [&](State &st, int k) {
            if (!st.ln.active) return;
            if (k < D) {
                const T *zk = zg + (long long)k * plane;
                NDC_UNROLL
                for (int n = 0; n < NZR; ++n)
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i)
                        st.pz[i][n] = *reinterpret_cast<const uint32_t *>(zk + i * cplane + st.zoff[n]);
            }
            const int kx = k - PD;
            if (kx >= 0 && kx < D) {
                const T *xk = xg + (long long)kx * plane;
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n)
                    st.px[n] = *reinterpret_cast<const uint32_t *>(xk + st.xoff[n]);
            } else {
                NDC_UNROLL
                for (int n = 0; n < NXR; ++n) st.px[n] = 0u;
            }
        };

        // registers -> LDS: source plane k as channel-pair words into slot k % 3; x plane
        // k - 1 completes the plane-pair word (x[k-2], x[k-1]) of slot (k - 2) % 3
        auto store_plane = [&](State &st, int k) {
            if (!st.ln.active) return;
            const int lb = PL + st.ln.c0;
            const int sb = off_s + wrap(k % NS, NS) * 2 * RS * P;
            const bool zin = k < D;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                if (!((st.zok >> n) & 1u)) continue;
                const int j = st.ln.strip + n * S;
                float s[SC][RW];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    s[i][0] = bf_lo(st.pz[i][n]) + st.bv[i];
                    s[i][1] = bf_hi(st.pz[i][n]) + st.bv[i];
                    if (relu) {
                        s[i][0] = relu_f(s[i][0]);
                        s[i][1] = relu_f(s[i][1]);
                    }
                }
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) {
                    const uint32_t w01 = zin ? pack_bf16x2(s[0][c], s[1][c]) : 0u;
                    const uint32_t w23 = zin ? pack_bf16x2(s[2][c], s[3][c]) : 0u;
                    ex.st_(sb + j * P + lb + c, bits_to_float(w01));
                    ex.st_(sb + (RS + j) * P + lb + c, bits_to_float(w23));
                }
            }
            const int xb = off_x + wrap((k - 2) % NX, NX) * RX * P;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                if ((st.xok >> n) & 1u) {
                    const int j = st.ln.strip + n * S;
                    ex.st_(xb + j * P + lb, bits_to_float(zip_lo(st.pxprev[n], st.px[n])));
                    ex.st_(xb + j * P + lb + 1, bits_to_float(zip_hi(st.pxprev[n], st.px[n])));
                }
                st.pxprev[n] = st.px[n];
            }
        };

        ex.each([&](State &st, int tid) {
            st.ln = make_lane(tid, t, RW);
            st.zok = st.xok = st.ook = 0u;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RS && row >= 0 && row < H) st.zok |= 1u << n;
                st.zoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) st.pz[i][n] = 0u;
            }
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX && row >= 0 && row < H) st.xok |= 1u << n;
                st.xoff[n] = clampi(row, 0, H - 1) * W + st.ln.c0;
                st.px[n] = st.pxprev[n] = 0u;
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
            for (int r = 0; r < RHK; ++r)
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) {
                    st.t1prev[r][c] = 0.f;
                    NDC_UNROLL
                    for (int a = 0; a < KD; ++a) st.t1acc[a][r][c] = 0.f;
                }
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        for (int k = 0; k < D + 2; ++k) {
            ex.each([&](State &st, int) { store_plane(st, k); });
            ex.sync();

            // ---- K-scatter of source plane k; own source words of plane k - 2; t1 plane k - 1
            ex.each([&](State &st, int) {
                if (!st.ln.active) return;
                const bool extra = st.ln.strip < 2;
                const int jx = halo_row(st.ln.strip, PH, TH);
                const int cb = PL + st.ln.c0 - PW;
                if (k < D) {
                    const int sb = off_s + wrap(k % NS, NS) * 2 * RS * P + cb;
                    float wp[KT], wn[KT];
                    load_taps<KT>(tab, wp);
                    NDC_ROLLED
                    for (int pr = 0; pr < 2; ++pr) {
                        load_taps<KT>(tab + uniform_int((pr + 1) & 1) * KT, wn);
                        const int b0 = sb + pr * RS * P;
                        k_rows_d2<RH, RW, RHK>(ex, b0 + (PH + st.ln.strip * RH) * P, P, wp, st.t1acc, 0);
                        if (extra) k_rows_d2<1, RW, RHK>(ex, b0 + jx * P, P, wp, st.t1acc, RH);
                        copy_taps<KT>(wn, wp);
                    }
                }
                if (k >= 2) {
                    const int ob = off_s + wrap((k - 2) % NS, NS) * 2 * RS * P + PL + st.ln.c0;
                    NDC_UNROLL
                    for (int pr = 0; pr < 2; ++pr)
                        NDC_UNROLL
                        for (int r = 0; r < RH; ++r)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c)
                                st.own[pr][r][c] = float_to_bits(
                                    ex.ld(ob + (pr * RS + 2 * PH + st.ln.strip * RH + r) * P + c));
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
                    float v[RW];
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        v[c] = live ? st.t1acc[0][r][c] : 0.f;
                        if (mine) ex.st_(tb + j * P + c, bits_to_float(pack_bf16x2(st.t1prev[r][c], v[c])));
                        st.t1prev[r][c] = v[c];
                    }
                    if (r < RH && t1g && live) IO::store(t1g + (long long)pf * plane + st.ooff[r < RH ? r : 0], v);
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        st.t1acc[0][r][c] = st.t1acc[1][r][c];
                        st.t1acc[1][r][c] = st.t1acc[2][r][c];
                        st.t1acc[2][r][c] = 0.f;
                    }
                }
            });
            ex.sync();

            // ---- prefetch, then A-gather + epilogue of plane k - 2
            ex.each([&](State &st, int) {
                if (!st.ln.active) return;
                load_plane(st, k + 1);
                const int j0 = k - 2;
                if (j0 < 0) return;
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
                for (int s = 0; s < 2; ++s) {
                    float wt[SC][9];
                    load_plane_taps<SC, 9, 9>(tab + 54 + s * 36, wt);
                    const int m = j0 - 1 + s;
                    const int ob = (st.ln.strip * RH) * P + PL + st.ln.c0 - PW;
                    const int base[2] = {off_x + wrap(m % NX, NX) * RX * P + ob,
                                         off_t + wrap(m % NTP, NTP) * RX * P + ob};
                    a_plane_d2<RH, RW, 2>(ex, base, P, wt, acc);
                }
                T *ok_ = og + (long long)j0 * plane;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (!((st.ook >> r) & 1u)) continue;
                    NDC_UNROLL
                    for (int i = 0; i < SC; ++i) {
                        float v[RW];
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) {
                            const uint32_t w = st.own[i >> 1][r][c];
                            const float s = (i & 1) ? bf_hi(w) : bf_lo(w);
                            v[c] = s * (acc[0][i][r][c] + eps) * fast_rcp(acc[1][i][r][c] + eps);
                        }
                        IO::store(ok_ + i * cplane + st.ooff[r], v);
                    }
                }
            });
        }
    }
};

}  // namespace fused
}  // namespace ndc
