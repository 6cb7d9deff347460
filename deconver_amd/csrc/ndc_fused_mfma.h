// bfloat16 kernels of the 3x3x3, SC = 4 depthwise geometry built on the 4x4x4 matrix
// instruction (mfma_bf16_4x4x4 in ndc_common.h): 1024 multiply-accumulates per wavefront
// instruction in about 10 clocks, where v_dot2c_f32_bf16 does 128 in 4.5.  Same work
// decomposition and march as ndc_fused_bf16.h (a thread owns RH rows x 2 columns); what
// changes is how the tap sums map to instructions.
//
//   K-type applications (4 -> 1 channels, scattered into the three pending output planes):
//     per (th, tw) one instruction per output voxel column,
//       D[m][n] += sum_i  H[m][i] * S[i][n],   H[m][i] = h[i][2 - m][th][tw]  (m = 3: zeros)
//     n = the lane's voxel, S[.][n] = its four source channels at the tap's neighbour,
//     D[m][n] = pending output plane m at the lane's voxel.  The source is staged as four
//     bf16 channels (8 bytes) per voxel; a thread reads the 4-voxel window of a row once
//     (two 16-byte reads) and picks the neighbour per tap from registers.  The tap rows H
//     sit in 18 registers per lane (lane & 3 selects the row m).
//
//   Filter-gradient terms  gh[i][tap] = sum_voxels g_i[v] * u[v + shift(tap)]  (g = gn or gd
//     with u = x or t1):  per (td, th) and 4-voxel group of a row
//       D[i][j] += sum_{k<4} g_i[c + k] * u[c + k + j - 1]        (j <-> tw = 2 - j)
//     lane (b, i) reads channel i of the staged g row (channel-major copy), lane (b, j) the
//     window of u starting at column c + j - 1.  LDS reads of 8 or 16 bytes must be aligned
//     to their size, so each u row is staged three times, shifted by -1, 0 and +1 column;
//     lane j reads copy j at the block's own (aligned) position.  The shifted words are made
//     from the lane's own column pair and its left neighbour's (one wavefront shift).
//     Each lane ends with the 9 x 4 sums of its block for ONE tw; the block reduction at the
//     end of the kernel adds lanes with equal (lane & 3).
//
// Both forms need whole 4-lane blocks inside one image row and a row inside one wavefront:
// W a multiple of 8 and W / 2 a divisor of 64.
#pragma once

#include "ndc_fused_bf16.h"

namespace ndc {
namespace fused {

// the smallest stride >= n words that is 16 modulo 64: rows of four channels (copies) that
// far apart put the four lanes of a block, which read them at one position, on different banks
NDC_HD int stride16(int n) { return (n + 47) / 64 * 64 + 16; }

// (hi half of `left`, lo half of `own`): the bf16 pair one column to the left of `own`
NDC_HD uint32_t shift_in_left(uint32_t own, uint32_t left) { return (left >> 16) | (own << 16); }

// =================================================================== forward (bf16, matrix instruction)

//   A-type applications (1 -> 4 channels): per (td, th) one instruction per output voxel column,
//       D[i][n] += sum_{k<4} T[i][k] * V[k][n],   T[i][k] = h[i][td][th][2 - k]  (k = 3: zero)
//     V[.][n] = the four columns n - 1 .. n + 2 of the operand's row.  A row is staged twice,
//     as bf16 pairs starting at the odd columns (copy 0, first pair (0, v[0])) and at the even
//     ones (copy 1): the window of the lane's even column is two consecutive words of copy 0,
//     that of its odd column two consecutive words of copy 1.
//
// out = s (A(x) + eps) / (A(K(s)) + eps); the pipeline is that of FwdKernelB: step k scatters
// source plane k into the three pending t1 planes and completes t1 plane k - 1 (phase 1), then
// gathers numerator and denominator of plane k - 2 and stages source plane k + 1 (phase 2).
template <int RH_> struct FwdKernelM {
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int kMinStrips = 4;
    static constexpr int RHK = RH + 1, NZR = RH + 1, NXR = RH + 1;
    static constexpr int NX = 3;   // ring slots of x and of t1 planes
    typedef bf16_t T;
    typedef FwdParams<T> Params;

    struct State {
        Lane ln;
        unsigned zoff[NZR], xoff[NXR], ooff[RH];
        unsigned zok, xok;
        MfmaRows wm[9], wg[9];
        f4_t t1acc[RHK][RW];
        uint32_t tq[RHK];       // the t1 plane just completed, own rows, as column pairs
        // staging registers, two sets: set (plane & 1) holds a source (x) plane from its fetch,
        // two steps before it is staged, until then.  The plane loop is unrolled twice, so the
        // sets are fixed registers.
        uint32_t pz[2][SC][NZR];
        uint32_t px[2][NXR];
    };

    static NDC_HD bool covers(int W) { return W % 8 == 0 && W <= 128 && 64 % (W / 2) == 0; }
    static NDC_HD int rows_s(int TH) { return TH + 4; }
    static NDC_HD int rows_x(int TH) { return TH + 2; }
    static NDC_HD int pitch_x(int W) { return W / 2 + 1; }   // one word past the row: (v[W-1], 0) / zeros
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int W = t.CPW * RW;
        return rows_s(t.TH) * 2 * t.P + 2 * NX * 2 * rows_x(t.TH) * pitch_x(W);
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int P2 = 2 * t.P, PX = pitch_x(W);
        const int RS = rows_s(TH), RX = rows_x(TH);
        const int CPS = RX * PX;                       // one staged copy of a plane
        const int off_s = 0, off_x = RS * P2, off_t = off_x + NX * 2 * CPS;
        const int total = off_t + NX * 2 * CPS;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef xb_ = make_buf(p.x + cbase, xbytes), zb_ = make_buf(p.z + cbase * SC, sbytes);
        const BufRef ob_ = make_buf(p.out + cbase * SC, sbytes);
        const BufRef tb_ = make_buf(p.t1 ? p.t1 + cbase : nullptr, xbytes);
        const BufRef db_ = make_buf(p.s_over_den ? p.s_over_den + cbase * SC : nullptr, sbytes);
        const BufRef rb_ = make_buf(p.ratio ? p.ratio + cbase * SC : nullptr, sbytes);
        const bool have_saved = p.s_over_den != nullptr;
        const float *tabm = p.wtab + (long long)id.c * kTabWords + kTabWM;
        const float *tabg = p.wtab + (long long)id.c * kTabWords + kTabWG;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();
        const float eps = p.eps;
        // the channel's four bias values: wave-uniform, fetched through the scalar unit
        float bv[SC];
        {
            UniformF bu = as_uniform(p.bias ? p.bias + id.c * SC : p.wtab);
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) bv[i] = p.bias ? bu[i] : 0.f;
        }

        // source plane k / x plane kx into staging set `set` (= the plane's parity)
        auto load_z = [&](State &st, int k, auto set_tag) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            // (planes past the end: a clamped plane is fetched and never staged; a branch
            // around the loads would keep the compiler from counting the outstanding ones)
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n)
                NDC_UNROLL
                for (int i = 0; i < SC; ++i)
                    st.pz[SET][i][n] = buf_ld(zb_, st.zoff[n], ko + i * cplane2);
        };
        auto load_x = [&](State &st, int kx, auto set_tag) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            // planes outside the volume: a clamped plane is loaded and zero selected
            const bool xlive = kx >= 0 && kx < D;
            const unsigned xk = (unsigned)clampi(kx, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const uint32_t v = buf_ld(xb_, st.xoff[n], xk);
                st.px[SET][n] = xlive ? v : 0u;
            }
        };
        // registers -> LDS: source plane k, four bf16 channels per voxel
        auto store_plane = [&](State &st, int k, auto set_tag) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            if (!st.ln.active) return;
            // planes past the end are never K-scattered, so the slot may keep stale words
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                if (k >= D || !((st.zok >> n) & 1u)) continue;
                const int j = st.ln.strip + n * S;
                float s[SC][RW];
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    s[i][0] = floor_f(bf_lo(st.pz[SET][i][n]) + bv[i], floor_);
                    s[i][1] = floor_f(bf_hi(st.pz[SET][i][n]) + bv[i], floor_);
                }
                const int o = off_s + j * P2 + (PL + st.ln.c0) * 2;
                NDC_UNROLL
                for (int c = 0; c < RW; ++c)
                    ex.st2(o + 2 * c, pack_bf16x2(s[0][c], s[1][c]), pack_bf16x2(s[2][c], s[3][c]));
            }
        };
        // a row of column pairs -> its two staged copies (`left`: the pair of the lane to the left)
        auto stage_row = [&](State &st, int at, uint32_t own, uint32_t left) NDC_LAMBDA {
            if (st.ln.c0 == 0) left = 0u;
            ex.stw(at, shift_in_left(own, left));
            ex.stw(at + CPS, own);
            if (st.ln.c0 == W - 2) ex.stw(at + 1, own >> 16);
        };
        // x plane k - 1 (fetched during the step before) -> ring slot (k - 1) % NX
        auto store_x = [&](State &st, int k, auto set_tag) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            const int kx = k - PD;
            const bool xlive = kx >= 0 && kx < D;
            const unsigned xk = (unsigned)clampi(kx, 0, D - 1) * plane2;
            const int xb = off_x + wrap(kx % NX, NX) * 2 * CPS + st.ln.c0 / 2;
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const uint32_t own = st.px[SET][n];
                const uint32_t left = from_left_lane(own, [&]() NDC_LAMBDA {
                    if (st.ln.c0 == 0 || st.xoff[n] >= kNoAccess || !xlive) return 0u;
                    return buf_ld(xb_, st.xoff[n] - 4u, xk);
                });
                if ((st.xok >> n) & 1u) stage_row(st, xb + (st.ln.strip + n * S) * PX, own, left);
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.zok = st.xok = 0u;
            NDC_UNROLL
            for (int n = 0; n < NZR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - 2 * PH + j;
                if (j < RS && row >= 0 && row < H) st.zok |= 1u << n;
                st.zoff[n] = st.ln.active ? (unsigned)(clampi(row, 0, H - 1) * W + st.ln.c0) * 2u : kNoAccess;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) st.pz[0][i][n] = st.pz[1][i][n] = 0u;
            }
            NDC_UNROLL
            for (int n = 0; n < NXR; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RX) st.xok |= 1u << n;
                st.xoff[n] = st.ln.active && j < RX && row >= 0 && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
                st.px[0][n] = st.px[1][n] = 0u;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                st.ooff[r] = row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
            }
            NDC_UNROLL
            for (int t9 = 0; t9 < 9; ++t9) {
                mfma_rows(st.wm[t9], tid, [&](int m, uint32_t (&w)[2]) NDC_LAMBDA {
                    w[0] = float_to_bits(tabm[(m * 9 + t9) * 2]);
                    w[1] = float_to_bits(tabm[(m * 9 + t9) * 2 + 1]);
                });
                mfma_rows(st.wg[t9], tid, [&](int m, uint32_t (&w)[2]) NDC_LAMBDA {
                    w[0] = float_to_bits(tabg[(m * 9 + t9) * 2]);
                    w[1] = float_to_bits(tabg[(m * 9 + t9) * 2 + 1]);
                });
            }
            const f4_t zero = {0.f, 0.f, 0.f, 0.f};
            NDC_UNROLL
            for (int r = 0; r < RHK; ++r) {
                st.tq[r] = 0u;
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) st.t1acc[r][c] = zero;
            }
            ex.wait_loads();
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_z(st, 0, IntTag<0>());
            load_x(st, 0, IntTag<0>());
        });
        ex.sync();
        ex.each([&](State &st, int) NDC_LAMBDA {
            store_plane(st, 0, IntTag<0>());
            load_z(st, 1, IntTag<1>());
        });
        ex.sync();

        // one plane step; PAR = k % 2, known at compile time (the loop below is unrolled twice)
        auto step = [&](int k, auto par_tag) NDC_LAMBDA {
            constexpr int PAR = decltype(par_tag)::value;

            // ---- x plane k - 1 staged; K-scatter of source plane k; t1 plane k - 1 completed
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (!st.ln.active) return;
                store_x(st, k, IntTag<1 - PAR>());
                const bool extra = st.ln.strip < 2;
                const int jx = halo_row(st.ln.strip, PH, TH);
                if (k < D) {
                    const int cb = off_s + (PL + st.ln.c0 - PW) * 2;
                    // the 4-voxel window of source row `at`, every tap of it that feeds the NR
                    // rows acc[r_off ...]; q = the window's row among the NR + 2 input rows
                    auto read_w = [&](int at, uint32_t (&v)[8]) NDC_LAMBDA {
                        uint32_t lo[4], hi[4];
                        ex.ld4a(at, lo);
                        ex.ld4a(at + 4, hi);
                        NDC_UNROLL
                        for (int u = 0; u < 4; ++u) {
                            v[u] = lo[u];
                            v[4 + u] = hi[u];
                        }
                    };
                    auto scatter = [&](int q, auto nr_tag, int r_off, const uint32_t (&v)[8]) NDC_LAMBDA {
                        constexpr int NR = decltype(nr_tag)::value;
                        NDC_UNROLL
                        for (int th = 0; th < KH; ++th) {
                            const int rr = q - th;
                            if (rr < 0 || rr >= NR) continue;
                            NDC_UNROLL
                            for (int tw = 0; tw < KW; ++tw)
                                NDC_UNROLL
                                for (int c = 0; c < RW; ++c)
                                    mfma_bf16_4x4x4(st.t1acc[r_off + rr][c], st.wm[th * 3 + tw],
                                                    v[(c + tw) * 2], v[(c + tw) * 2 + 1]);
                        }
                    };
                    const int b0 = cb + (PH + st.ln.strip * RH) * P2;
                    uint32_t kv[2][8];
                    read_w(b0, kv[0]);
                    NDC_UNROLL
                    for (int q = 0; q < RH + 2; ++q) {
                        if (q + 1 < RH + 2) read_w(b0 + (q + 1) * P2, kv[(q + 1) & 1]);
                        ex.fence();
                        scatter(q, IntTag<RH>(), 0, kv[q & 1]);
                        ex.fence();
                    }
                    if (extra) {
                        const int b1 = cb + jx * P2;
                        NDC_UNROLL
                        for (int q = 0; q < 3; ++q) {
                            uint32_t v[8];
                            read_w(b1 + q * P2, v);
                            scatter(q, IntTag<1>(), RH, v);
                        }
                    }
                }
                // t1 plane k - 1 is complete: to ring slot (k - 1) % NX and to global memory
                const int pf = k - PD;
                const bool inplane = pf >= 0 && pf < D;
                const int tb = off_t + wrap(pf % NX, NX) * 2 * CPS + st.ln.c0 / 2;
                NDC_UNROLL
                for (int r = 0; r < RHK; ++r) {
                    const bool mine = r < RH || extra;
                    const int j = r < RH ? PH + st.ln.strip * RH + r : jx;
                    const int row = r0 - PH + j;
                    const bool live = inplane && row >= 0 && row < H;
                    const uint32_t vq = live ? pack_bf16x2(st.t1acc[r][0][0], st.t1acc[r][1][0]) : 0u;
                    st.tq[r] = vq;
                    const uint32_t left = ex.left_lane([&](State &o) NDC_LAMBDA { return o.tq[r]; });
                    if (mine) stage_row(st, tb + j * PX, vq, left);
                    if (r < RH && live) buf_st(tb_, st.ooff[r < RH ? r : 0], (unsigned)pf * plane2, vq);
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c)
                        st.t1acc[r][c] = f4_t{st.t1acc[r][c][1], st.t1acc[r][c][2], 0.f, 0.f};
                }
            });
            ex.sync();

            // ---- prefetch, then A-gather + epilogue of plane k - 2, then staging of plane k + 1
            ex.each([&](State &st, int) NDC_LAMBDA {
                // fetched now, staged two steps on: source plane k + 2, x plane k + 1
            // (every lane issues every fetch, lanes outside the tile with offsets outside the
            // slices: a fetch under a condition gives the compiler a path without it, on which
            // it cannot count the outstanding loads, and then every use of a prefetched
            // register waits for ALL loads)
                load_z(st, k + 2, IntTag<PAR>());
                load_x(st, k + 1, IntTag<1 - PAR>());
                if (!st.ln.active) return;
                const int j0 = k - 2;
                if (j0 < 0 || j0 >= D) {
                    store_plane(st, k + 1, IntTag<1 - PAR>());
                    return;
                }
                // the own source values of plane j0: z is read again (staged two steps ago: L2)
                uint32_t own[SC][RH];
                f4_t acc[2][RH][RW];   // numerator, denominator; four channels each
                NDC_UNROLL
                for (int a = 0; a < 2; ++a)
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) acc[a][r][c] = f4_t{eps, eps, eps, eps};
                {
                    const int lc = st.ln.c0 / 2;
                    // unit u = (operand, td, row pair): the windows of two of the RH + 2 rows of
                    // plane j0 + 1 - td; read two units ahead of the instructions that use them
                    static_assert(RH == 2, "the units below pair the RH + 2 = 4 input rows");
                    auto read_a = [&](int u, uint32_t (&v)[2][RW][2]) NDC_LAMBDA {
                        const int op = u / (2 * KD), td = (u / 2) % KD, q0 = (u % 2) * 2;
                        const int at = (op ? off_t : off_x) + wrap((j0 + 1 - td) % NX, NX) * 2 * CPS +
                                       (st.ln.strip * RH + q0) * PX + lc;
                        NDC_UNROLL
                        for (int q = 0; q < 2; ++q)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) ex.ld2w(at + c * CPS + q * PX, v[q][c]);
                    };
                    auto mfma_a = [&](int u, const uint32_t (&v)[2][RW][2]) NDC_LAMBDA {
                        const int op = u / (2 * KD), td = (u / 2) % KD, q0 = (u % 2) * 2;
                        NDC_UNROLL
                        for (int q = 0; q < 2; ++q)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r) {
                                const int th = r + 2 - (q0 + q);
                                if (th < 0 || th >= KH) continue;
                                NDC_UNROLL
                                for (int c = 0; c < RW; ++c)
                                    mfma_bf16_4x4x4(acc[op][r][c], st.wg[td * 3 + th], v[q][c][0], v[q][c][1]);
                            }
                    };
                    constexpr int NU = 2 * KD * 2;
                    uint32_t av[3][2][RW][2];
                    read_a(0, av[0]);
                    read_a(1, av[1]);
                    NDC_UNROLL
                    for (int u = 0; u < NU; ++u) {
                        if (u + 2 < NU) read_a(u + 2, av[(u + 2) % 3]);
                        if (u == NU - 3) {
                            // (issued here, when the last windows have been requested: before
                            // the loop they would hold eight more registers through it)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r)
                                NDC_UNROLL
                                for (int i = 0; i < SC; ++i)
                                    own[i][r] = buf_ld(zb_, st.ooff[r], (unsigned)j0 * plane2 + i * cplane2);
                        }
                        ex.fence();
                        mfma_a(u, av[u % 3]);
                        ex.fence();
                    }
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
                            // same arithmetic as the staging: the staged value before its rounding
                            const float s = floor_f((c ? bf_hi(w) : bf_lo(w)) + bv[i], floor_);
                            const float inv = fast_rcp(acc[1][r][c][i]);
                            rd[c] = s * inv;
                            rt[c] = acc[0][r][c][i] * inv;
                            v[c] = s * rt[c];
                        }
                        buf_st<true>(ob_, st.ooff[r], oj + i * cplane2, pack_bf16x2(v[0], v[1]));
                        if (have_saved) {
                            buf_st<true>(db_, st.ooff[r], oj + i * cplane2, pack_bf16x2(rd[0], rd[1]));
                            buf_st<true>(rb_, st.ooff[r], oj + i * cplane2, pack_bf16x2(rt[0], rt[1]));
                        }
                    }
                }
                store_plane(st, k + 1, IntTag<1 - PAR>());
            });
            ex.sync();
        };
        // An even number of steps, the last possibly one past the end of the march (it finds
        // nothing to do): with the second step of an iteration under a condition the compiler
        // sees a path from one even step straight to the next and, unable to count the loads
        // outstanding on it, makes every use of a prefetched register wait for all loads.
        for (int kk = 0; kk < D + 2; kk += 2) {
            step(uniform_int(kk), IntTag<0>());
            step(uniform_int(kk + 1), IntTag<1>());
        }
    }
};

// =================================================================== backward pass 1 (bf16, matrix instruction)

// Reads the forward's s/d and n/d (the form every training step uses): gn = g s/d,
// gd = -gn n/d, gx = K(gn), gt1 = K(gd), and the A-side filter-gradient terms.
template <int RH_> struct Bwd1KernelM {
    static constexpr bool SAVED = true;
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int NXS = RH + 1;   // x / t1 rows a thread stages (the last: first two strips)
    static constexpr int NX = 3;         // ring slots of x / t1 planes
    static constexpr int NRED = SC * KT;
    typedef bf16_t T;
    typedef BwdParams<T> Params;

    struct State {
        Lane ln;
        int lane4, blk4;      // lane & 3; first word of the lane's block in a row of pairs
        unsigned xoff[NXS], ooff[RH], hoff;
        unsigned xok;
        MfmaRows wm[9];
        f4_t accx[RH][RW], acct[RH][RW];
        f4_t gacc[KD][KH];
        uint32_t px[NXS], pt[NXS];
        // gout, s/d, n/d words of two planes: set (plane & 1) holds a plane from its fetch, two
        // steps before it is used, until then (the plane loop is unrolled twice: fixed registers)
        uint32_t qg[2][SC][RH + 1], qd[2][SC][RH + 1], qr[2][SC][RH + 1];
    };

    static NDC_HD bool covers(int W) { return W % 8 == 0 && W <= 128 && 64 % (W / 2) == 0; }
    static NDC_HD int rows_g(int TH) { return TH + 2; }
    // strides of the channel rows of the channel-major copy and of the shifted copies: a
    // multiple of 64 words plus 16, so that the four lanes of a block, which read four
    // different channels (copies) at one position, hit different banks
    static NDC_HD int stride_gc(int TH, int W) { return stride16(TH * (W / 2)); }
    static NDC_HD int stride_xs(int TH, int W) { return stride16((TH + 2) * (W / 2)); }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int W = t.CPW * RW;
        const int main_ = 2 * rows_g(t.TH) * 2 * t.P + 2 * SC * stride_gc(t.TH, W) +
                          NX * 2 * 3 * stride_xs(t.TH, W);
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, PL = t.PL, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int P2 = 2 * t.P, WH = W / 2;
        const int RG = rows_g(TH), RXS = TH + 2;
        const int GCS = stride_gc(TH, W), XCS = stride_xs(TH, W);
        const int off_gp = 0, off_gc = 2 * RG * P2, off_xs = off_gc + 2 * SC * GCS;
        const int total = off_xs + NX * 2 * 3 * XCS;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef xb_ = make_buf(p.x + cbase, xbytes), tb_ = make_buf(p.t1 + cbase, xbytes);
        const BufRef gb_ = make_buf(p.gout + cbase * SC, sbytes);
        const BufRef db_ = make_buf(p.s_over_den + cbase * SC, sbytes);
        const BufRef rb_ = make_buf(p.ratio + cbase * SC, sbytes);
        const BufRef gxb_ = make_buf(p.gx ? p.gx + cbase : nullptr, xbytes);
        const BufRef gtb_ = make_buf(p.gt1 + cbase, xbytes);
        const float *tabm = p.wtab + (long long)id.c * kTabWords + kTabWM;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const int need_gh = p.need_gh;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                const uint32_t vx = buf_ld(xb_, st.xoff[n], ko);
                const uint32_t vt = buf_ld(tb_, st.xoff[n], ko);
                st.px[n] = live ? vx : 0u;
                st.pt[n] = live ? vt : 0u;
            }
        };
        // plane k of x and t1 (in the registers since load_plane) goes to ring slot k % 3 as
        // three copies per row: pairs starting one column left of the even columns (copy 0),
        // at them (copy 1), one column right of them (copy 2)
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int slot = wrap(k % NX, NX);
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                NDC_UNROLL
                for (int op = 0; op < 2; ++op) {
                    const uint32_t own = op ? st.pt[n] : st.px[n];
                    uint32_t left = from_left_lane(own, [&]() NDC_LAMBDA {
                        if (st.ln.c0 == 0 || st.xoff[n] >= kNoAccess || !live) return 0u;
                        return buf_ld(op ? tb_ : xb_, st.xoff[n] - 4u, ko);
                    });
                    if (st.ln.c0 == 0) left = 0u;
                    const uint32_t sh = shift_in_left(own, left);
                    if ((st.xok >> n) & 1u) {
                        const int row = off_xs + (slot * 2 + op) * 3 * XCS +
                                        (st.ln.strip + n * S) * WH + st.ln.c0 / 2;
                        ex.stw(row, sh);
                        ex.stw(row + XCS, own);
                        if (st.ln.c0 > 0) ex.stw(row + 2 * XCS - 1, sh);
                        if (st.ln.c0 == W - 2) ex.stw(row + 2 * XCS, own >> 16);
                    }
                }
            }
        };
        // gout, s/d, n/d words of plane jn into the state, a phase before they are used (own
        // rows, then the halo row of the first two strips)
        auto prefetch_g = [&](State &st, int jn, auto set_tag) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            // (no branch around the loads, also past the last plane, where a clamped plane is
            // fetched and never used: with loads on one path only the compiler cannot count
            // the outstanding ones, and makes the next user of ANY load wait for all)
            const unsigned jo = (unsigned)clampi(jn, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int r = 0; r < RH + 1; ++r) {
                if (r == RH && st.ln.strip >= 2) continue;
                const unsigned o = r < RH ? st.ooff[r < RH ? r : 0] : st.hoff;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    st.qg[SET][i][r] = buf_ld<true>(gb_, o, jo + i * cplane2);
                    st.qd[SET][i][r] = buf_ld<true>(db_, o, jo + i * cplane2);
                    st.qr[SET][i][r] = buf_ld<true>(rb_, o, jo + i * cplane2);
                }
            }
        };
        // gn, gd of the prefetched row `pr` -> tile row j of the per-voxel copy (four channels
        // per voxel) and, for own rows, row `own` of the channel-major copy
        auto publish_row = [&](State &st, auto set_tag, int pr, int j, int own) NDC_LAMBDA {
            constexpr int SET = decltype(set_tag)::value;
            float gn[SC][RW], gd[SC][RW];
            NDC_UNROLL
            for (int i = 0; i < SC; ++i)
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) {
                    // (the words of a row outside the image were read as zeros)
                    const float gv = c ? bf_hi(st.qg[SET][i][pr]) : bf_lo(st.qg[SET][i][pr]);
                    gn[i][c] = gv * (c ? bf_hi(st.qd[SET][i][pr]) : bf_lo(st.qd[SET][i][pr]));
                    gd[i][c] = -(gn[i][c] * (c ? bf_hi(st.qr[SET][i][pr]) : bf_lo(st.qr[SET][i][pr])));
                }
            const int o = off_gp + j * P2 + (PL + st.ln.c0) * 2;
            NDC_UNROLL
            for (int c = 0; c < RW; ++c) {
                ex.st2(o + 2 * c, pack_bf16x2(gn[0][c], gn[1][c]), pack_bf16x2(gn[2][c], gn[3][c]));
                ex.st2(o + RG * P2 + 2 * c, pack_bf16x2(gd[0][c], gd[1][c]),
                       pack_bf16x2(gd[2][c], gd[3][c]));
            }
            if (own >= 0) {
                const int oc = off_gc + own * WH + st.ln.c0 / 2;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    ex.stw(oc + i * GCS, pack_bf16x2(gn[i][0], gn[i][1]));
                    ex.stw(oc + (SC + i) * GCS, pack_bf16x2(gd[i][0], gd[i][1]));
                }
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.lane4 = tid & 3;
            st.blk4 = (st.ln.c0 / 8) * 4;
            st.xok = 0u;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RXS) st.xok |= 1u << n;
                st.xoff[n] = st.ln.active && j < RXS && row >= 0 && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
                st.px[n] = st.pt[n] = 0u;
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
                    for (int r = 0; r < RH + 1; ++r)
                        NDC_UNROLL
                        for (int a = 0; a < 2; ++a) st.qg[a][i][r] = st.qd[a][i][r] = st.qr[a][i][r] = 0u;
            }
            NDC_UNROLL
            for (int t9 = 0; t9 < 9; ++t9)
                mfma_rows(st.wm[t9], tid, [&](int m, uint32_t (&w)[2]) NDC_LAMBDA {
                    w[0] = float_to_bits(tabm[(m * 9 + t9) * 2]);
                    w[1] = float_to_bits(tabm[(m * 9 + t9) * 2 + 1]);
                });
            const f4_t zero = {0.f, 0.f, 0.f, 0.f};
            NDC_UNROLL
            for (int r = 0; r < RH; ++r)
                NDC_UNROLL
                for (int c = 0; c < RW; ++c) st.accx[r][c] = st.acct[r][c] = zero;
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int b = 0; b < KH; ++b) st.gacc[a][b] = zero;
            // the tap rows have arrived before the march starts (otherwise every step's first
            // matrix instruction is made to wait for the loads issued just before it)
            ex.wait_loads();
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
            prefetch_g(st, 0, IntTag<0>());
        });
        ex.sync();

        // Two barriers per plane step.  Phase 1 of step k stages plane k of x / t1 (fetched
        // during the step before), fetches the next, and publishes gn / gd of plane k - 1;
        // phase 2 fetches gout, s/d, n/d of plane k + 1 and does all tap sums of plane k - 1.
        // one plane step; PAR = k % 2, known at compile time (the loop below is unrolled twice)
        auto step = [&](int k, auto par_tag) NDC_LAMBDA {
            constexpr int PAR = decltype(par_tag)::value;
            const int j1 = k - 1;
            const bool live1 = j1 >= 0 && j1 < D;
            ex.each([&](State &st, int) NDC_LAMBDA {
                if (st.ln.active) store_plane(st, k);
                // (x and t1 are fetched again as soon as consumed: they are needed at the start
                // of the next step; every lane issues every fetch, see below)
                load_plane(st, k + 1);
                if (!st.ln.active || !live1) return;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r)
                    publish_row(st, IntTag<1 - PAR>(), r, PH + st.ln.strip * RH + r, st.ln.strip * RH + r);
                if (st.ln.strip < 2) publish_row(st, IntTag<1 - PAR>(), RH, halo_row(st.ln.strip, PH, TH), -1);
            });
            ex.sync();

            ex.each([&](State &st, int) NDC_LAMBDA {
                // (every lane issues every fetch, lanes outside the tile with offsets outside
                // the slices: a fetch under a condition gives the compiler a path without it, on
                // which it cannot count the outstanding loads, and then every use of a
                // prefetched register waits for ALL loads)
                prefetch_g(st, k + 1, IntTag<1 - PAR>());
                if (!st.ln.active) return;
                if (live1) {
                    // LDS reads run ahead of the matrix instructions that use them (two
                    // wavefronts per SIMD do not hide their latency): the K-type rows two
                    // rows ahead, the filter-gradient rows a whole tap plane ahead.  The
                    // scheduling fences keep that order.
                    const int kbase = off_gp + (st.ln.strip * RH) * P2 + (PL + st.ln.c0 - PW) * 2;
                    // K-type group g = (kind, input row q): the 4-voxel window of gn (gd)
                    auto read_k = [&](int g, uint32_t (&v)[8]) NDC_LAMBDA {
                        const int at = kbase + ((g / (RH + 2)) * RG + g % (RH + 2)) * P2;
                        uint32_t lo[4], hi[4];
                        ex.ld4a(at, lo);
                        ex.ld4a(at + 4, hi);
                        NDC_UNROLL
                        for (int u = 0; u < 4; ++u) {
                            v[u] = lo[u];
                            v[4 + u] = hi[u];
                        }
                    };
                    // gn rows feed gx, gd rows feed gt1
                    auto mfma_k = [&](int g, const uint32_t (&v)[8]) NDC_LAMBDA {
                        const int kind = g / (RH + 2), q = g % (RH + 2);
                        NDC_UNROLL
                        for (int th = 0; th < KH; ++th) {
                            const int rr = q - th;
                            if (rr < 0 || rr >= RH) continue;
                            NDC_UNROLL
                            for (int tw = 0; tw < KW; ++tw)
                                NDC_UNROLL
                                for (int c = 0; c < RW; ++c)
                                    mfma_bf16_4x4x4(kind ? st.acct[rr][c] : st.accx[rr][c],
                                                    st.wm[th * 3 + tw], v[(c + tw) * 2],
                                                    v[(c + tw) * 2 + 1]);
                        }
                    };
                    // filter-gradient unit u = (operand, td, row pair): two of the RH + 2 rows of x
                    // (t1) of plane j1 + 1 - td around the own rows, in the lane's shifted copy
                    const int copy = st.lane4 < 3 ? st.lane4 : 1;
                    auto read_g = [&](int u, uint32_t (&bw)[2][4]) NDC_LAMBDA {
                        const int op = u / (2 * KD), td = (u / 2) % KD, q0 = (u % 2) * 2;
                        const int slot = wrap((j1 + 1 - td) % NX, NX);
                        const int xb = off_xs + ((slot * 2 + op) * 3 + copy) * XCS +
                                       (st.ln.strip * RH + q0) * WH + st.blk4;
                        NDC_UNROLL
                        for (int q = 0; q < 2; ++q) ex.ld4a(xb + q * WH, bw[q]);
                    };
                    // the block's 8 columns of gn (gd), channel = lane & 3, own rows
                    MfmaRows ga[2][RH][2];
                    auto read_ga = [&]() NDC_LAMBDA {
                        NDC_UNROLL
                        for (int op = 0; op < 2; ++op)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r) {
                                const int at = off_gc + op * SC * GCS + (st.ln.strip * RH + r) * WH + st.blk4;
                                mfma_rows2(ga[op][r][0], ga[op][r][1], st.lane4,
                                           [&](int m, uint32_t (&w4)[4]) NDC_LAMBDA { ex.ld4a(at + m * GCS, w4); });
                            }
                    };
                    auto mfma_g = [&](int u, const uint32_t (&bw)[2][4]) NDC_LAMBDA {
                        const int op = u / (2 * KD), td = (u / 2) % KD, q0 = (u % 2) * 2;
                        NDC_UNROLL
                        for (int q = 0; q < 2; ++q)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r) {
                                const int th = r + 2 - (q0 + q);
                                if (th < 0 || th >= KH) continue;
                                mfma_bf16_4x4x4(st.gacc[td][th], ga[op][r][0], bw[q][0], bw[q][1]);
                                mfma_bf16_4x4x4(st.gacc[td][th], ga[op][r][1], bw[q][2], bw[q][3]);
                            }
                    };
                    static_assert(RH == 2, "the units pair the RH + 2 = 4 input rows");
                    constexpr int NKG = 2 * (RH + 2), NGG = 2 * KD * 2;
                    uint32_t kv[2][8];
                    uint32_t bw[3][2][4];
                    read_k(0, kv[0]);
                    NDC_UNROLL
                    for (int g = 0; g < NKG; ++g) {
                        if (g + 1 < NKG) read_k(g + 1, kv[(g + 1) & 1]);
                        if (need_gh && g + 2 == NKG) read_ga();
                        if (need_gh && g + 1 == NKG) {
                            read_g(0, bw[0]);
                            read_g(1, bw[1]);
                        }
                        ex.fence();
                        mfma_k(g, kv[g & 1]);
                        ex.fence();
                    }
                    if (need_gh) {
                        NDC_UNROLL
                        for (int g = 0; g < NGG; ++g) {
                            if (g + 2 < NGG) read_g(g + 2, bw[(g + 2) % 3]);
                            ex.fence();
                            mfma_g(g, bw[g % 3]);
                            ex.fence();
                        }
                    }
                }
                const int pf = k - 2;
                NDC_UNROLL
                for (int r = 0; r < RH; ++r) {
                    if (pf >= 0 && pf < D) {   // rows outside the image: the stores go nowhere
                        buf_st<true>(gxb_, st.ooff[r], (unsigned)pf * plane2,
                                     pack_bf16x2(st.accx[r][0][0], st.accx[r][1][0]));
                        buf_st(gtb_, st.ooff[r], (unsigned)pf * plane2,
                               pack_bf16x2(st.acct[r][0][0], st.acct[r][1][0]));
                    }
                    NDC_UNROLL
                    for (int c = 0; c < RW; ++c) {
                        st.accx[r][c] = f4_t{st.accx[r][c][1], st.accx[r][c][2], 0.f, 0.f};
                        st.acct[r][c] = f4_t{st.acct[r][c][1], st.acct[r][c][2], 0.f, 0.f};
                    }
                }
            });
            ex.sync();
        };
        // (an even number of steps, see FwdKernelM)
        for (int kk = 0; kk < D + 2; kk += 2) {
            step(uniform_int(kk), IntTag<0>());
            step(uniform_int(kk + 1), IntTag<1>());
        }

        if (need_gh) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            // element (i, td, th, tw) is summed over the lanes whose window shift is 1 - tw
            ex.template block_reduce<NRED>(
                [](State &st, int e) NDC_LAMBDA {
                    const int i = e / KT, tap = e % KT, tw = tap % 3;
                    return st.lane4 == 2 - tw ? st.gacc[tap / 9][(tap % 9) / 3][i] : 0.f;
                },
                [&](int e, float v) NDC_LAMBDA { dst[e] = v; });
        }
    }
};

// =================================================================== backward pass 2 (bf16, matrix instruction)

//   A-type applications (1 -> 4 channels): per (td, th) one instruction per output voxel column,
//       D[i][n] += sum_{k<4} T[i][k] * V[k][n],   T[i][k] = h[i][td][th][2 - k]  (k = 3: zero)
//     V[.][n] = the four columns n - 1 .. n + 2 of the operand's row: two words of the copy
//     shifted by -1 column for the lane's even column, of the unshifted copy for its odd one.
//
// Reads the forward's n/d: gz = [s > 0] (g n/d + A(gt1)), gb, and the K-side filter-gradient
// term sum_v s_i[v] gt1[v + shift(tap)], in the block form described at the top of this file
// (lane (b, i) reads channel i of the staged s row).  One barrier per plane step: the step of
// plane j0 stages s of plane j0 channel-major in one of two buffers, and the filter-gradient
// instructions of that plane run a step later, after the barrier; the gt1 ring therefore
// holds five planes.
template <int RH_> struct Bwd2KernelM {
    static constexpr bool SAVED = true;
    static constexpr int KD = 3, KH = 3, KW = 3, SC = 4, RH = RH_, RW = 2;
    static constexpr int PD = 1, PH = 1, PW = 1, KT = 27;
    static constexpr int NXS = RH + 1;
    static constexpr int NG = 5;   // ring slots of gt1 planes
    static constexpr int NRED = SC * KT + SC;
    typedef bf16_t T;
    typedef BwdParams<T> Params;

    struct State {
        Lane ln;
        int lane4, blk4;
        unsigned xoff[NXS], ooff[RH];
        unsigned xok;
        float bvr[SC][RH];
        float okf[RH];
        MfmaRows wg[9];
        f4_t gacc[KD][KH];
        float gbacc[SC];
        uint32_t pg[NXS];
        // the z, gout, n/d words of two planes: the step of plane parity P consumes set 1 - P
        // (fetched at the start of the step before) and starts the fetch of its own plane's
        // into set P, so a fetch has more than a whole step to arrive.  The plane loop is
        // unrolled twice: the sets are fixed registers.
        uint32_t qz[2][SC][RH], qg[2][SC][RH], qr[2][SC][RH];
    };

    // (below 32 columns the dot2 kernel is the faster one: measured 0.095 against 0.134 ms at
    // 512 channels of 16^3)
    static NDC_HD bool covers(int W) { return W % 8 == 0 && W >= 32 && W <= 128 && 64 % (W / 2) == 0; }
    static NDC_HD int pitch_xs(int W) { return W / 2 + 4; }   // one zero word past the row, rows 16-byte aligned
    static NDC_HD int stride_xs(int TH, int W) { return stride16((TH + 2) * pitch_xs(W)); }
    static NDC_HD int stride_sc(int TH, int W) { return stride16(TH * (W / 2)); }
    static NDC_HD int lds_floats(const Tile &t)
    {
        const int W = t.CPW * RW;
        const int main_ = NG * 3 * stride_xs(t.TH, W) + 2 * SC * stride_sc(t.TH, W);
        const int red = (t.NT / 64) * NRED;
        return main_ > red ? main_ : red;
    }

    template <class Exec> static NDC_D void run(Exec &ex, const Params &p, int block_id)
    {
        const Tile t = p.t;
        const BlockId id = decode_block(block_id, p.C, t, p.D);
        const int S = t.S, TH = t.TH, W = p.W, H = p.H, D = p.D;
        const int WH = W / 2, PX = pitch_xs(W), RXS = TH + 2;
        const int XCS = stride_xs(TH, W), SCS = stride_sc(TH, W);
        const int off_xs = 0, off_sc = NG * 3 * XCS;
        const int total = off_sc + 2 * SC * SCS;
        const int plane = H * W;
        const long long cplane = (long long)D * plane;
        const long long cbase = ((long long)id.b * p.C + id.c) * cplane;
        const size_t xbytes = (size_t)cplane * sizeof(T), sbytes = xbytes * SC;
        const unsigned plane2 = (unsigned)plane * 2u, cplane2 = (unsigned)cplane * 2u;
        const BufRef gtb_ = make_buf(p.gt1 + cbase, xbytes);
        const BufRef zb_ = make_buf(p.z + cbase * SC, sbytes), gb_ = make_buf(p.gout + cbase * SC, sbytes);
        const BufRef rb_ = make_buf(p.ratio + cbase * SC, sbytes);
        const BufRef gzb_ = make_buf(p.gz ? p.gz + cbase * SC : nullptr, sbytes);
        const float *tabg = p.wtab + (long long)id.c * kTabWords + kTabWG;
        const int r0 = id.r0;
        const int nthreads = ex.nthreads;
        const float floor_ = p.relu ? 0.f : pass_through_floor();
        const int need_gh = p.need_gh;
        const int relu = p.relu;

        auto load_plane = [&](State &st, int k) NDC_LAMBDA {
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                const uint32_t vg = buf_ld(gtb_, st.xoff[n], ko);
                st.pg[n] = live ? vg : 0u;
            }
        };
        // plane k of gt1 -> ring slot k % NG as three copies per row (see Bwd1KernelM)
        auto store_plane = [&](State &st, int k) NDC_LAMBDA {
            if (!st.ln.active) return;
            const int slot = wrap(k % NG, NG);
            const bool live = k < D;
            const unsigned ko = (unsigned)clampi(k, 0, D - 1) * plane2;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                const uint32_t own = st.pg[n];
                uint32_t left = from_left_lane(own, [&]() NDC_LAMBDA {
                    if (st.ln.c0 == 0 || st.xoff[n] >= kNoAccess || !live) return 0u;
                    return buf_ld(gtb_, st.xoff[n] - 4u, ko);
                });
                if (st.ln.c0 == 0) left = 0u;
                const uint32_t sh = shift_in_left(own, left);
                if ((st.xok >> n) & 1u) {
                    const int row = off_xs + slot * 3 * XCS + (st.ln.strip + n * S) * PX + st.ln.c0 / 2;
                    ex.stw(row, sh);
                    ex.stw(row + XCS, own);
                    if (st.ln.c0 > 0) ex.stw(row + 2 * XCS - 1, sh);
                    if (st.ln.c0 == W - 2) {
                        ex.stw(row + 2 * XCS, own >> 16);
                        ex.stw(row + 1, own >> 16);
                    }
                }
            }
        };

        ex.each([&](State &st, int tid) NDC_LAMBDA {
            st.ln = make_lane(tid, t, RW);
            st.lane4 = tid & 3;
            st.blk4 = (st.ln.c0 / 8) * 4;
            st.xok = 0u;
            NDC_UNROLL
            for (int n = 0; n < NXS; ++n) {
                const int j = st.ln.strip + n * S, row = r0 - PH + j;
                if (j < RXS) st.xok |= 1u << n;
                st.xoff[n] = st.ln.active && j < RXS && row >= 0 && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
                st.pg[n] = 0u;
            }
            NDC_UNROLL
            for (int r = 0; r < RH; ++r) {
                const int row = r0 + st.ln.strip * RH + r;
                st.ooff[r] = st.ln.active && row < H ? (unsigned)(row * W + st.ln.c0) * 2u : kNoAccess;
                st.okf[r] = row < H ? 1.f : 0.f;
                NDC_UNROLL
                for (int i = 0; i < SC; ++i) {
                    // a row outside the image reads zeros; -1 (rectified) or 0 makes its source 0
                    st.bvr[i][r] = row < H ? (p.bias ? p.bias[id.c * SC + i] : 0.f) : (p.relu ? -1.f : 0.f);
                    st.qz[0][i][r] = st.qg[0][i][r] = st.qr[0][i][r] = 0u;
                    st.qz[1][i][r] = st.qg[1][i][r] = st.qr[1][i][r] = 0u;
                }
            }
            NDC_UNROLL
            for (int t9 = 0; t9 < 9; ++t9)
                mfma_rows(st.wg[t9], tid, [&](int m, uint32_t (&w)[2]) NDC_LAMBDA {
                    w[0] = float_to_bits(tabg[(m * 9 + t9) * 2]);
                    w[1] = float_to_bits(tabg[(m * 9 + t9) * 2 + 1]);
                });
            const f4_t zero = {0.f, 0.f, 0.f, 0.f};
            NDC_UNROLL
            for (int a = 0; a < KD; ++a)
                NDC_UNROLL
                for (int b = 0; b < KH; ++b) st.gacc[a][b] = zero;
            NDC_UNROLL
            for (int i = 0; i < SC; ++i) st.gbacc[i] = 0.f;
            ex.wait_loads();
            for (int i = tid; i < total; i += nthreads) ex.st_(i, 0.f);
            load_plane(st, 0);
        });
        ex.sync();

        // one plane step; PAR = k % 2, known at compile time (the loop below is unrolled twice)
        auto compute = [&](State &st, int k, auto par_tag) NDC_LAMBDA {
                constexpr int PAR = decltype(par_tag)::value;
                const int j0 = k - 1;
                // (every lane issues every fetch, lanes outside the tile with offsets outside the
                // slices: a fetch under a condition gives the compiler a path without it, on which
                // it cannot count the outstanding loads, and then every use of a prefetched
                // register waits for ALL loads)
                load_plane(st, k + 1);
                // plane k's z, gout, n/d words, consumed by the next step
                {
                    const unsigned jn = (unsigned)clampi(k, 0, D - 1) * plane2;
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int i = 0; i < SC; ++i) {
                            st.qz[PAR][i][r] = buf_ld(zb_, st.ooff[r], jn + i * cplane2);
                            st.qg[PAR][i][r] = buf_ld<true>(gb_, st.ooff[r], jn + i * cplane2);
                            st.qr[PAR][i][r] = buf_ld<true>(rb_, st.ooff[r], jn + i * cplane2);
                        }
                }
                if (!st.ln.active) return;
                const int lc = st.ln.c0 / 2;
                if (j0 >= 0 && j0 < D) {
                    // A(gt1) of plane j0: windows of plane j0 + 1 - td, read a tap plane ahead
                    f4_t acc[RH][RW];
                    const f4_t zero = {0.f, 0.f, 0.f, 0.f};
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int c = 0; c < RW; ++c) acc[r][c] = zero;
                    auto read_a = [&](int td, uint32_t (&v)[RH + 2][RW][2]) NDC_LAMBDA {
                        const int slot = wrap((j0 + 1 - td) % NG, NG);
                        const int at = off_xs + slot * 3 * XCS + (st.ln.strip * RH) * PX + lc;
                        NDC_UNROLL
                        for (int q = 0; q < RH + 2; ++q)
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) ex.ld2w(at + c * XCS + q * PX, v[q][c]);
                    };
                    auto mfma_a = [&](int td, const uint32_t (&v)[RH + 2][RW][2]) NDC_LAMBDA {
                        NDC_UNROLL
                        for (int q = 0; q < RH + 2; ++q)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r) {
                                const int th = r + 2 - q;
                                if (th < 0 || th >= KH) continue;
                                NDC_UNROLL
                                for (int c = 0; c < RW; ++c)
                                    mfma_bf16_4x4x4(acc[r][c], st.wg[td * 3 + th], v[q][c][0], v[q][c][1]);
                            }
                    };
                    uint32_t av[2][RH + 2][RW][2];
                    read_a(0, av[0]);
                    NDC_UNROLL
                    for (int td = 0; td < KD; ++td) {
                        if (td + 1 < KD) read_a(td + 1, av[(td + 1) & 1]);
                        ex.fence();
                        mfma_a(td, av[td & 1]);
                        ex.fence();
                    }
                    // gz, gb; s of this plane to the channel-major buffer k & 1
                    const unsigned jo = (unsigned)j0 * plane2;
                    const int osc = off_sc + (k & 1) * SC * SCS + (st.ln.strip * RH) * WH + lc;
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r)
                        NDC_UNROLL
                        for (int i = 0; i < SC; ++i) {
                            float v[RW], sv[RW];
                            NDC_UNROLL
                            for (int c = 0; c < RW; ++c) {
                                const float s = floor_f((c ? bf_hi(st.qz[1 - PAR][i][r]) : bf_lo(st.qz[1 - PAR][i][r])) + st.bvr[i][r], floor_);
                                const float g = c ? bf_hi(st.qg[1 - PAR][i][r]) : bf_lo(st.qg[1 - PAR][i][r]);
                                float gzv = g * (c ? bf_hi(st.qr[1 - PAR][i][r]) : bf_lo(st.qr[1 - PAR][i][r])) + acc[r][c][i];
                                if (relu && s <= 0.f) gzv = 0.f;   // a NaN passes
                                sv[c] = s;
                                st.gbacc[i] += gzv * st.okf[r];
                                v[c] = gzv;
                            }
                            buf_st<true>(gzb_, st.ooff[r], jo + i * cplane2, pack_bf16x2(v[0], v[1]));
                            ex.stw(osc + i * SCS + r * WH, pack_bf16x2(sv[0], sv[1]));
                        }
                }
                const int js = j0 - 1;   // the plane whose s was staged a step ago
                if (need_gh && js >= 0 && js < D) {
                    const int copy = st.lane4 < 3 ? st.lane4 : 1;
                    MfmaRows ga[RH][2];
                    NDC_UNROLL
                    for (int r = 0; r < RH; ++r) {
                        const int at = off_sc + ((k - 1) & 1) * SC * SCS + (st.ln.strip * RH + r) * WH + st.blk4;
                        mfma_rows2(ga[r][0], ga[r][1], st.lane4,
                                   [&](int m, uint32_t (&w4)[4]) NDC_LAMBDA { ex.ld4a(at + m * SCS, w4); });
                    }
                    auto read_g = [&](int td, uint32_t (&bw)[RH + 2][4]) NDC_LAMBDA {
                        const int slot = wrap((js + 1 - td) % NG, NG);
                        const int xb = off_xs + (slot * 3 + copy) * XCS + (st.ln.strip * RH) * PX + st.blk4;
                        NDC_UNROLL
                        for (int q = 0; q < RH + 2; ++q) ex.ld4a(xb + q * PX, bw[q]);
                    };
                    auto mfma_g = [&](int td, const uint32_t (&bw)[RH + 2][4]) NDC_LAMBDA {
                        NDC_UNROLL
                        for (int q = 0; q < RH + 2; ++q)
                            NDC_UNROLL
                            for (int r = 0; r < RH; ++r) {
                                const int th = r + 2 - q;
                                if (th < 0 || th >= KH) continue;
                                mfma_bf16_4x4x4(st.gacc[td][th], ga[r][0], bw[q][0], bw[q][1]);
                                mfma_bf16_4x4x4(st.gacc[td][th], ga[r][1], bw[q][2], bw[q][3]);
                            }
                    };
                    uint32_t bw[2][RH + 2][4];
                    read_g(0, bw[0]);
                    NDC_UNROLL
                    for (int td = 0; td < KD; ++td) {
                        if (td + 1 < KD) read_g(td + 1, bw[(td + 1) & 1]);
                        ex.fence();
                        mfma_g(td, bw[td & 1]);
                        ex.fence();
                    }
                }
        };
        for (int kk = 0; kk < D + 2; kk += 2) {
            {
                const int k = uniform_int(kk);
                ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k); });
                ex.sync();
                ex.each([&](State &st, int) NDC_LAMBDA { compute(st, k, IntTag<0>()); });
            }
            {   // (an even number of steps, see FwdKernelM)
                const int k = uniform_int(kk + 1);
                ex.each([&](State &st, int) NDC_LAMBDA { store_plane(st, k); });
                ex.sync();
                ex.each([&](State &st, int) NDC_LAMBDA { compute(st, k, IntTag<1>()); });
            }
        }

        if (p.need_gh || p.need_gb) {
            float *dst = p.part + (long long)block_id * p.part_stride;
            ex.template block_reduce<NRED>(
                [](State &st, int e) NDC_LAMBDA {
                    if (e >= SC * KT) return st.gbacc[e >= SC * KT ? e - SC * KT : 0];
                    const int i = e / KT, tap = e % KT, tw = tap % 3;
                    return st.lane4 == 2 - tw ? st.gacc[tap / 9][(tap % 9) / 3][i < SC ? i : 0] : 0.f;
                },
                [&](int e, float v) NDC_LAMBDA { dst[e] = v; });
        }
    }
};

}  // namespace fused
}  // namespace ndc
