// Sequential host build of the NDC C ABI.  Same kernel bodies and host logic as the HIP
// build, executed thread by thread on the CPU, so that the CPU test-suite can check
// indexing, bounds and barrier placement before anything runs on a GPU.  It is a checker
// for the kernels' source, not a fallback: the Python package never loads it.
#include <cmath>
#include <vector>

#include "ndc_common.h"
#include "ndc_exec.h"

#define NDC_LAMBDA

namespace ndc {

struct NoTimer {
    NoTimer(bool, void *) {}
    void mark() {}
    void finish(float *ms, int count)
    {
        if (ms) for (int i = 0; i < count; ++i) ms[i] = 0.f;
    }
};

struct Backend {
    static constexpr bool is_device = false;
    static constexpr int kSumSlices = 8;
    typedef NoTimer Timer;

    template <class Kernel>
    static int block_kernel(const typename Kernel::Params &p, int nblocks, int nthreads,
                            int lds_floats, void *)
    {
        for (int blk = 0; blk < nblocks; ++blk) {
            HostExec<typename Kernel::State> ex(nthreads, lds_floats);
            Kernel::run(ex, p, blk);
        }
        return 0;
    }

    template <class F> static int elementwise(long long n, void *, F f)
    {
        for (long long idx = 0; idx < n; ++idx) f(idx);
        return 0;
    }

    static int transpose(const void *src, void *dst, long long batch, long long R, long long K,
                         int esz, void *)
    {
        const char *s = (const char *)src;
        char *d = (char *)dst;
        for (long long b = 0; b < batch; ++b)
            for (long long r = 0; r < R; ++r)
                for (long long k = 0; k < K; ++k)
                    memcpy(d + ((b * K + k) * R + r) * esz, s + ((b * R + r) * K + k) * esz, (size_t)esz);
        return 0;
    }

    // Row normalisation as the HIP build computes it (part by part, float32 sums, the same
    // shift and the same formulas), sequentially.
    template <typename T>
    static void rownorm_t(bool bwd, const T *a, const T *b, const T *addend, float *partial, float *stats,
                          T *out, long long rows, long long n, int nsplit, long long chunk, float eps)
    {
        for (long long row = 0; row < rows; ++row) {
            const T *ar = a + row * n, *br = bwd ? b + row * n : nullptr;
            float pivot = 0.f;
            if (!bwd) {
                const long long first = n < 256 ? n : 256;
                for (long long i = 0; i < first; ++i) pivot += Elem<T>::load(ar + i);
                pivot /= (float)first;
            }
            float s1 = 0.f, s2 = 0.f, cnt = 0.f, mean = 0.f, m2 = 0.f;
            for (int part = 0; part < nsplit; ++part) {
                const long long lo = part * chunk, hi = lo + chunk < n ? lo + chunk : n;
                float p1 = 0.f, p2 = 0.f;
                for (long long i = lo; i < hi; ++i) {
                    const float f = Elem<T>::load(ar + i) - pivot;
                    p1 += f;
                    p2 += f * (bwd ? Elem<T>::load(br + i) : f);
                }
                const float np = (float)(hi - lo);
                if (!bwd) {
                    // the part's (mean, squared deviations), merged into the row's
                    const float pm = pivot + p1 / np, pq = p2 - p1 * p1 / np;
                    partial[2 * (row * nsplit + part)] = pm;
                    partial[2 * (row * nsplit + part) + 1] = pq;
                    const float tot = cnt + np, delta = pm - mean;
                    mean += delta * (np / tot);
                    m2 += pq + delta * delta * (cnt * np / tot);
                    cnt = tot;
                } else {
                    partial[2 * (row * nsplit + part)] = p1;
                    partial[2 * (row * nsplit + part) + 1] = p2;
                    s1 += p1;
                    s2 += p2;
                }
            }
            const float inv_n = 1.f / (float)n;
            float c0, c1, c2 = 0.f;
            if (bwd) {
                c1 = stats[2 * row + 1];
                c0 = -c1 * s1 * inv_n;
                c2 = -c1 * s2 * inv_n;
            } else {
                float var = m2 * inv_n;
                var = var > 0.f ? var : 0.f;
                c1 = 1.f / std::sqrt(var + eps);
                c0 = mean;
                stats[2 * row] = c0;
                stats[2 * row + 1] = c1;
            }
            for (long long i = 0; i < n; ++i) {
                const float v = Elem<T>::load(ar + i);
                float f = bwd ? v * c1 + c0 + Elem<T>::load(br + i) * c2 : (v - c0) * c1;
                if (bwd && addend) f += Elem<T>::load(addend + row * n + i);
                Elem<T>::store(out + row * n + i, f);
            }
        }
    }

    static int rownorm(bool bwd, const void *a, const void *b, const void *addend, float *partial, float *stats,
                       void *out, long long rows, long long n, int nsplit, long long chunk, int esz, bool,
                       float eps, void *)
    {
        if (esz == 2)
            rownorm_t<bf16_t>(bwd, (const bf16_t *)a, (const bf16_t *)b, (const bf16_t *)addend, partial, stats,
                              (bf16_t *)out, rows, n, nsplit, chunk, eps);
        else
            rownorm_t<float>(bwd, (const float *)a, (const float *)b, (const float *)addend, partial, stats,
                             (float *)out, rows, n, nsplit, chunk, eps);
        return 0;
    }

    static int regroup2(const void *src, void *dst, const float *bias, long long rows, int channels, int D,
                        int H, int W, int depth2, int esz, int to_channels, void *)
    {
        const int Dc = depth2 ? D / 2 : 1, Hc = H / 2, Wc = W / 2, nk = depth2 ? 8 : 4;
        const long long plane = (long long)Dc * Hc * Wc;
        for (long long r = 0; r < rows; ++r)
            for (int d = 0; d < D; ++d)
                for (int h = 0; h < H; ++h)
                    for (int w = 0; w < W; ++w) {
                        const int kd = depth2 ? (d & 1) : 0, k = (kd * 2 + (h & 1)) * 2 + (w & 1);
                        const long long fine = ((r * D + d) * H + h) * (long long)W + w;
                        const long long coarse =
                            (r * nk + k) * plane + ((long long)(depth2 ? d / 2 : 0) * Hc + h / 2) * Wc + w / 2;
                        if (to_channels) {
                            memcpy((char *)dst + coarse * esz, (const char *)src + fine * esz, (size_t)esz);
                        } else if (esz == 2) {
                            const float v = Elem<bf16_t>::load((const bf16_t *)src + coarse);
                            Elem<bf16_t>::store((bf16_t *)dst + fine, bias ? v + bias[r % channels] : v);
                        } else {
                            const float v = ((const float *)src)[coarse];
                            ((float *)dst)[fine] = bias ? v + bias[r % channels] : v;
                        }
                    }
        return 0;
    }

    // normalisation over channels, sequentially, with the HIP build's partial-sum layout (one
    // partial row per wavefront of 64 x (16 / esz or 1) voxels)
    static constexpr int kChnormWaves = 4;
    static long long chnorm_blocks(long long n, int esz, bool vec)
    {
        const long long per = vec ? 16 / esz : 1;
        return (n / per + 255) / 256;
    }
    template <typename T>
    static void chnorm_t(bool bwd, const T *a, const T *x, float *stats, const float *weight, const float *bias,
                         T *out, float *partial, long long B, int C, long long n, bool vec, float eps)
    {
        const long long per = vec ? 16 / (long long)sizeof(T) : 1, blocks = chnorm_blocks(n, (int)sizeof(T), vec);
        if (bwd && partial)
            for (long long k = 0; k < B * blocks * kChnormWaves * C * 2; ++k) partial[k] = 0.f;
        for (long long b = 0; b < B; ++b)
            for (long long i = 0; i < n; ++i) {
                const T *xb = x + b * C * n + i;
                if (!bwd) {
                    float mean = 0.f, m2 = 0.f;
                    for (int c = 0; c < C; ++c) {
                        const float v = Elem<T>::load(xb + c * n), d = v - mean;
                        mean += d * (1.f / (float)(c + 1));
                        m2 += d * (v - mean);
                    }
                    const float rstd = 1.f / std::sqrt(m2 / (float)C + eps);
                    stats[(b * 2 + 0) * n + i] = mean;
                    stats[(b * 2 + 1) * n + i] = rstd;
                    for (int c = 0; c < C; ++c)
                        Elem<T>::store(out + b * C * n + c * n + i,
                                       (Elem<T>::load(xb + c * n) - mean) * rstd * (weight ? weight[c] : 1.f) +
                                           (bias ? bias[c] : 0.f));
                } else {
                    const T *gb = a + b * C * n + i;
                    const float mean = stats[(b * 2 + 0) * n + i], rstd = stats[(b * 2 + 1) * n + i];
                    const long long wave = (b * blocks + i / per / 256) * kChnormWaves + (i / per % 256) / 64;
                    float s1 = 0.f, s2 = 0.f;
                    for (int c = 0; c < C; ++c) {
                        const float g = Elem<T>::load(gb + c * n), w = weight ? weight[c] : 1.f;
                        const float xh = (Elem<T>::load(xb + c * n) - mean) * rstd;
                        s1 += g * w;
                        s2 += g * w * xh;
                        if (partial) {
                            partial[(wave * C + c) * 2] += g * xh;
                            partial[(wave * C + c) * 2 + 1] += g;
                        }
                    }
                    for (int c = 0; c < C; ++c) {
                        const float g = Elem<T>::load(gb + c * n), w = weight ? weight[c] : 1.f;
                        const float xh = (Elem<T>::load(xb + c * n) - mean) * rstd;
                        Elem<T>::store(out + b * C * n + c * n + i, rstd * (g * w - s1 / (float)C - xh * s2 / (float)C));
                    }
                }
            }
    }
    static int chnorm(bool bwd, const void *a, const void *x, const float *stats, const float *weight,
                      const float *bias, void *out, float *partial, long long B, int C, long long n, int esz,
                      bool vec, float eps, void *)
    {
        if (esz == 2)
            chnorm_t<bf16_t>(bwd, (const bf16_t *)a, (const bf16_t *)x, const_cast<float *>(stats), weight, bias,
                             (bf16_t *)out, partial, B, C, n, vec, eps);
        else
            chnorm_t<float>(bwd, (const float *)a, (const float *)x, const_cast<float *>(stats), weight, bias,
                            (float *)out, partial, B, C, n, vec, eps);
        return 0;
    }

    static int row_sums(const void *a, float *partial, long long rows, long long n, int nsplit, long long chunk,
                        int esz, bool, void *)
    {
        for (long long row = 0; row < rows; ++row)
            for (int part = 0; part < nsplit; ++part) {
                const long long lo = part * chunk, hi = lo + chunk < n ? lo + chunk : n;
                float s = 0.f;
                for (long long i = row * n + lo; i < row * n + hi; ++i)
                    s += esz == 2 ? Elem<bf16_t>::load((const bf16_t *)a + i) : ((const float *)a)[i];
                partial[row * nsplit + part] = s;
            }
        return 0;
    }

    static float act_value(int act, float u, bool grad)
    {
        const float cdf = 0.5f * (1.f + std::erf(u * 0.70710678118654752f));
        if (act == 1) return grad ? (u > 0.f ? 1.f : 0.f) : (u > 0.f ? u : 0.f);
        if (act == 2) return grad ? cdf + u * 0.3989422804014327f * std::exp(-0.5f * u * u) : u * cdf;
        return grad ? 1.f : u;
    }

    // the packed weights of the streaming GEMM: fragment (c, s), lane l, element e holds
    // W[32 c + l % 32][16 s + 8 (l / 32) + e] as bf16
    static int pwgemm_pack(const void *w, int w_is_bf16, int transposed, void *wfrag, int cout, int cin, void *)
    {
        const int S = cin / 16;
        bf16_t *o = (bf16_t *)wfrag;
        for (int c = 0; c < cout / 32; ++c)
            for (int s = 0; s < S; ++s)
                for (int l = 0; l < 64; ++l)
                    for (int e = 0; e < 8; ++e) {
                        const int row = 32 * c + l % 32, k = 16 * s + 8 * (l / 32) + e;
                        const long long at = transposed ? (long long)k * cout + row : (long long)row * cin + k;
                        const float v = w_is_bf16 ? Elem<bf16_t>::load((const bf16_t *)w + at) : ((const float *)w)[at];
                        o[(((long long)c * S + s) * 64 + l) * 8 + e] = float_to_bf16(v);
                    }
        return 0;
    }

    static int pwgemm(const void *x, const void *wfrag, const float *bias, const void *res, void *y, void *zkeep,
                      float *gpart, const void *mask, long long batch, int cin, int cout, long long n, int act, void *)
    {
        if (gpart)
            for (long long i = 0; i < 4096LL * cout; ++i) gpart[i] = 0.f;
        const int S = cin / 16;
        const bf16_t *xs = (const bf16_t *)x, *wf = (const bf16_t *)wfrag, *rs = (const bf16_t *)res;
        bf16_t *ys = (bf16_t *)y, *zs = (bf16_t *)zkeep;
        for (long long b = 0; b < batch; ++b)
            for (int co = 0; co < cout; ++co)
                for (long long v = 0; v < n; ++v) {
                    float acc = 0.f;
                    for (int k = 0; k < cin; ++k) {
                        const long long f = ((long long)(co / 32) * S + k / 16) * 64 + (k % 16 / 8) * 32 + co % 32;
                        acc += Elem<bf16_t>::load(wf + f * 8 + k % 8) * Elem<bf16_t>::load(xs + (b * cin + k) * n + v);
                    }
                    const long long at = (b * cout + co) * n + v;
                    if (act == 3 || act == 4) {   // times the derivative of relu (3) / gelu (4) at aux + bias
                        const float out = acc * act_value(act - 2, Elem<bf16_t>::load(rs + at) + (bias ? bias[co] : 0.f), true);
                        if (gpart) gpart[(v / 64 % 7) * cout + co] += out;   // a few rows, as the device uses many
                        ys[at] = float_to_bf16(out);
                        continue;
                    }
                    if (act == 5) {   // the sum where mask > 0, else 0
                        float out = acc + (bias ? bias[co] : 0.f) + (rs ? Elem<bf16_t>::load(rs + at) : 0.f);
                        if (!(Elem<bf16_t>::load((const bf16_t *)mask + at) > 0.f)) out = 0.f;
                        ys[at] = float_to_bf16(out);
                        continue;
                    }
                    if (zs) zs[at] = float_to_bf16(acc);
                    float out = act_value(act, acc + (bias ? bias[co] : 0.f), false);
                    if (rs) out += Elem<bf16_t>::load(rs + at);
                    ys[at] = float_to_bf16(out);
                }
        return 0;
    }

    template <typename T>
    static void bias_act_t(const T *z, const float *bias, const T *res, T *y, long long rows, int channels,
                           long long n, int act)
    {
        for (long long row = 0; row < rows; ++row) {
            const float b = bias ? bias[row % channels] : 0.f;
            for (long long i = row * n; i < (row + 1) * n; ++i)
                Elem<T>::store(y + i, act_value(act, Elem<T>::load(z + i) + b, false) + (res ? Elem<T>::load(res + i) : 0.f));
        }
    }

    static int bias_act(const void *z, const float *bias, const void *res, void *y, long long rows,
                        int channels, long long n, int, long long, int act, int esz, bool, void *)
    {
        if (esz == 2) bias_act_t<bf16_t>((const bf16_t *)z, bias, (const bf16_t *)res, (bf16_t *)y, rows, channels, n, act);
        else bias_act_t<float>((const float *)z, bias, (const float *)res, (float *)y, rows, channels, n, act);
        return 0;
    }

    template <typename T>
    static void bias_act_bwd_t(const T *gy, const T *z, const float *bias, T *gz, float *gpart, long long rows,
                               int channels, long long n, int nsplit, long long chunk, int act)
    {
        for (long long row = 0; row < rows; ++row) {
            const float b = bias ? bias[row % channels] : 0.f;
            for (int part = 0; part < nsplit; ++part) {
                const long long lo = part * chunk, hi = lo + chunk < n ? lo + chunk : n;
                float s = 0.f;
                for (long long i = row * n + lo; i < row * n + hi; ++i) {
                    const float v = Elem<T>::load(gy + i) * act_value(act, Elem<T>::load(z + i) + b, true);
                    s += v;
                    Elem<T>::store(gz + i, v);
                }
                if (gpart) gpart[row * nsplit + part] = s;
            }
        }
    }

    static int bias_act_backward(const void *gy, const void *z, const float *bias, void *gz, float *gpart,
                                 long long rows, int channels, long long n, int nsplit, long long chunk, int act,
                                 int esz, bool, void *)
    {
        if (esz == 2)
            bias_act_bwd_t<bf16_t>((const bf16_t *)gy, (const bf16_t *)z, bias, (bf16_t *)gz, gpart, rows, channels, n,
                                   nsplit, chunk, act);
        else
            bias_act_bwd_t<float>((const float *)gy, (const float *)z, bias, (float *)gz, gpart, rows, channels, n,
                                  nsplit, chunk, act);
        return 0;
    }

    // put(o, sum_p term(o, p)) in the association of the HIP build (kSumSlices interleaved
    // partial sums, then those in order)
    template <class P, class F> static int strided_sum(int nout, int nparts, void *, P put, F term)
    {
        for (int o = 0; o < nout; ++o) {
            float total = 0.f;
            for (int j = 0; j < kSumSlices; ++j) {
                float acc = 0.f;
                for (int p = j; p < nparts; p += kSumSlices) acc += term(o, p);
                total += acc;
            }
            put(o, total);
        }
        return 0;
    }

    template <class F> static int block_reduce(int nout, void *, float *out, F partial)
    {
        float buf[256];
        for (int o = 0; o < nout; ++o) {
            for (int tid = 0; tid < 256; ++tid) buf[tid] = partial(o, tid, 256);
            for (int s = 128; s > 0; s >>= 1)
                for (int tid = 0; tid < s; ++tid) buf[tid] += buf[tid + s];
            out[o] = buf[0];
        }
        return 0;
    }
};

}  // namespace ndc

#include "ndc_api_impl.h"

// LDS faults (races, out-of-bounds, uninitialised reads) seen by the host execution since
// the last call; `first` describes the first one.  Test hook of the host build only.
extern "C" long long ndc_host_faults(char *first, int n)
{
    ndc::HostFaults &f = ndc::host_faults();
    const long long total = f.races + f.oob + f.uninit;
    if (first && n > 0) {
        snprintf(first, (size_t)n, "%s", f.first);
    }
    f = ndc::HostFaults();
    return total;
}
