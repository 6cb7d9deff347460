// What follows a 1x1 projection in a Deconver block, in one pass over its output: the
// per-channel bias, the activation and the residual sum,
//
//   y[b][c][i] = act(z[b][c][i] + bias[c]) + residual[b][c][i]        act: none | relu | gelu
//
// on channel-first tensors (B, C, n), i.e. B*C contiguous rows of n elements, and the gradient
// of the activation with the bias gradient's partial sums,
//
//   gz = gy * act'(z + bias),   gpart[row][part] = sum over the part of gz.
//
// PyTorch runs these as a broadcast add, an activation and a residual add: three passes that
// read and write the tensor (the mixer's out_proj and the MLP's two projections,
// deconver.py:41-46, 60-64; layers/mlp.py:40-63 of the reference).  Rows are cut into parts as
// for the row normalisation.  float32 arithmetic, 16-byte accesses.  Device code only.
#pragma once
#include "ndc_rownorm.h"

namespace ndc {
namespace epilogue {

using rownorm::kThreads;
using rownorm::Split;
using rownorm::Vec;

enum { kNone = 0, kRelu = 1, kGelu = 2 };

// erf(x) and exp(-x^2) together (Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7: one reciprocal,
// one exponential, a degree-5 polynomial).  The library erff costs about twice as many
// instructions, which is what bounds these passes once their memory accesses are 16 bytes wide.
__device__ inline float erf_and_gauss(float x, float &gauss)
{
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(1.f + 0.3275911f * ax);
    gauss = __expf(-ax * ax);
    const float poly =
        t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    return copysignf(1.f - poly * gauss, x);
}

template <int ACT> __device__ inline float act_fwd(float u)
{
    if (ACT == kRelu) return u > 0.f ? u : 0.f;
    if (ACT == kGelu) {
        float gauss;
        return 0.5f * u * (1.f + erf_and_gauss(u * 0.70710678118654752f, gauss));
    }
    return u;
}

template <int ACT> __device__ inline float act_grad(float u)
{
    if (ACT == kRelu) return u > 0.f ? 1.f : 0.f;
    if (ACT == kGelu) {
        float gauss;   // exp(-u^2 / 2)
        const float cdf = 0.5f * (1.f + erf_and_gauss(u * 0.70710678118654752f, gauss));
        return cdf + u * 0.3989422804014327f * gauss;
    }
    return 1.f;
}

// out = f(a, b) element by element over one part of a row; returns the part's sum of out in
// thread 0 when SUM
template <typename T, bool TWO, bool VEC, bool SUM, class F>
__device__ inline float map_part(const T *ar, const T *br, T *orow, long long lo, long long hi, F f)
{
    float total = 0.f;
    if constexpr (VEC) {
        typedef Vec<T> V;
        const V *av = reinterpret_cast<const V *>(ar), *bv = reinterpret_cast<const V *>(br);
        V *ov = reinterpret_cast<V *>(orow);
        const long long v0 = lo / V::N, v1 = hi / V::N;
        auto one = [&](const V &x, const V &y) {
            V r;
            float v[V::N];
#pragma unroll
            for (int e = 0; e < V::N; ++e) {
                v[e] = f(x.get(e), TWO ? y.get(e) : 0.f);
                if (SUM) total += v[e];
            }
            if constexpr (sizeof(T) == 2) {
#pragma unroll
                for (int p = 0; p < V::N / 2; ++p) r.set_pair(p, v[2 * p], v[2 * p + 1]);
            } else {
#pragma unroll
                for (int e = 0; e < V::N; ++e) r.set(e, v[e]);
            }
            return r;
        };
        long long i = v0 + threadIdx.x;
        for (; i + 3 * kThreads < v1; i += 4 * kThreads) {
            V x[4], y[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                x[u] = av[i + u * kThreads];
                if (TWO) y[u] = bv[i + u * kThreads];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) ov[i + u * kThreads] = one(x[u], y[u]);
        }
        for (; i < v1; i += kThreads) {
            const V x = av[i];
            V y;
            if (TWO) y = bv[i];
            ov[i] = one(x, y);
        }
    } else {
        for (long long i = lo + threadIdx.x; i < hi; i += kThreads) {
            const float v = f(Elem<T>::load(ar + i), TWO ? Elem<T>::load(br + i) : 0.f);
            if (SUM) total += v;
            Elem<T>::store(orow + i, v);
        }
    }
    return total;
}

template <typename T, int ACT, bool RES, bool VEC>
__global__ void __launch_bounds__(kThreads)
forward_kernel(const T *z, const float *bias, const T *residual, T *y, int channels, Split sp)
{
    const long long row = blockIdx.x / sp.nsplit;
    const int part = blockIdx.x % sp.nsplit;
    const float b = bias ? bias[row % channels] : 0.f;
    const long long lo = part * sp.chunk, hi = lo + sp.chunk < sp.n ? lo + sp.chunk : sp.n;
    map_part<T, RES, VEC, false>(z + row * sp.n, RES ? residual + row * sp.n : nullptr, y + row * sp.n, lo, hi,
                                 [b](float zv, float rv) { return act_fwd<ACT>(zv + b) + rv; });
}

template <typename T, int ACT, bool VEC>
__global__ void __launch_bounds__(kThreads)
backward_kernel(const T *gy, const T *z, const float *bias, T *gz, float *gpart, int channels, Split sp)
{
    __shared__ float buf[4][2];
    const long long row = blockIdx.x / sp.nsplit;
    const int part = blockIdx.x % sp.nsplit;
    const float b = bias ? bias[row % channels] : 0.f;
    const long long lo = part * sp.chunk, hi = lo + sp.chunk < sp.n ? lo + sp.chunk : sp.n;
    float s = map_part<T, true, VEC, true>(gy + row * sp.n, z + row * sp.n, gz + row * sp.n, lo, hi,
                                           [b](float g, float zv) { return g * act_grad<ACT>(zv + b); });
    float unused = 0.f;
    rownorm::block_sum2(s, unused, buf);
    if (gpart && threadIdx.x == 0) gpart[blockIdx.x] = s;
}

}  // namespace epilogue
}  // namespace ndc
