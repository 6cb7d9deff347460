// Normalisation over the CHANNEL axis of a channel-first tensor (B, C, n): for every voxel,
//   y[b][c][i] = (x[b][c][i] - mean[b][i]) * rstd[b][i] * weight[c] + bias[c]
// with mean and (biased) variance taken over c.  This is the reference's LayerNorm
// (deconver/layers/norm.py:25-34: nn.LayerNorm applied with the channel axis moved last) on the
// layout the tensors already have: lanes run along the voxels (16 bytes each), a loop runs over
// the channels, so every access is a contiguous run and nothing is transposed.
//
//   forward : loop 1 keeps a running mean and sum of squared deviations per voxel (Welford);
//             loop 2 reads x again and writes y.  stats[b][0][i] = mean, stats[b][1][i] = rstd.
//   backward: loop 1 sums g w and g w xhat per voxel and, per channel, g xhat and g over the
//             wavefront's voxels (partial[wave][c] = (sum g xhat, sum g): the affine gradients
//             are their sums over the wavefronts); loop 2 writes
//             gx = rstd (g w - mean_c(g w) - xhat mean_c(g w xhat)).
//
// HBM traffic: forward 2 reads + 1 write of the tensor, backward 4 reads + 1 write (the second
// read of a loop pair finds part of the tensor in the last-level cache).  float32 arithmetic.
// Device code only.
#pragma once
#include "ndc_rownorm.h"

namespace ndc {
namespace chnorm {

using rownorm::kThreads;
using rownorm::Vec;

struct Shape {
    long long n;      // voxels per (sample, channel)
    int channels;
    int blocks;       // workgroups per sample
};

template <typename T, bool VEC> struct Lanes {
    static constexpr int N = VEC ? Vec<T>::N : 1;
    float v[N];
    __device__ void load(const T *p)
    {
        if constexpr (VEC) {
            const Vec<T> x = *reinterpret_cast<const Vec<T> *>(p);
#pragma unroll
            for (int e = 0; e < N; ++e) v[e] = x.get(e);
        } else {
            v[0] = Elem<T>::load(p);
        }
    }
    __device__ void store(T *p) const
    {
        if constexpr (VEC) {
            Vec<T> r;
            if constexpr (sizeof(T) == 2) {
#pragma unroll
                for (int q = 0; q < N / 2; ++q) r.set_pair(q, v[2 * q], v[2 * q + 1]);
            } else {
#pragma unroll
                for (int e = 0; e < N; ++e) r.set(e, v[e]);
            }
            *reinterpret_cast<Vec<T> *>(p) = r;
        } else {
            Elem<T>::store(p, v[0]);
        }
    }
};

template <typename T, bool VEC>
__global__ void __launch_bounds__(kThreads)
forward_kernel(const T *x, const float *weight, const float *bias, T *y, float *stats, Shape s, float eps)
{
    typedef Lanes<T, VEC> L;
    const long long b = blockIdx.x / s.blocks;
    const long long i = ((long long)(blockIdx.x % s.blocks) * kThreads + threadIdx.x) * L::N;
    if (i >= s.n) return;
    const T *xb = x + b * s.channels * s.n + i;
    T *yb = y + b * s.channels * s.n + i;
    L t;
    // running mean and squared deviations per voxel (Welford): no cancellation whatever the
    // offset of the values
    float mean[L::N], m2[L::N];
#pragma unroll
    for (int e = 0; e < L::N; ++e) mean[e] = m2[e] = 0.f;
    for (int c = 0; c < s.channels; ++c) {
        t.load(xb + c * s.n);
        const float rk = 1.f / (float)(c + 1);
#pragma unroll
        for (int e = 0; e < L::N; ++e) {
            const float d = t.v[e] - mean[e];
            mean[e] += d * rk;
            m2[e] += d * (t.v[e] - mean[e]);
        }
    }
    const float inv_c = 1.f / (float)s.channels;
    float rstd[L::N];
#pragma unroll
    for (int e = 0; e < L::N; ++e) {
        rstd[e] = 1.f / sqrtf(m2[e] * inv_c + eps);
        stats[(b * 2 + 0) * s.n + i + e] = mean[e];
        stats[(b * 2 + 1) * s.n + i + e] = rstd[e];
    }
    for (int c = 0; c < s.channels; ++c) {
        const float w = weight ? weight[c] : 1.f, bb = bias ? bias[c] : 0.f;
        t.load(xb + c * s.n);
#pragma unroll
        for (int e = 0; e < L::N; ++e) t.v[e] = (t.v[e] - mean[e]) * rstd[e] * w + bb;
        t.store(yb + c * s.n);
    }
}

// partial: (gridDim.x * wavefronts per workgroup, channels, 2) floats, or null
template <typename T, bool VEC>
__global__ void __launch_bounds__(kThreads)
backward_kernel(const T *gy, const T *x, const float *stats, const float *weight, T *gx, float *partial,
                Shape s)
{
    typedef Lanes<T, VEC> L;
    const long long b = blockIdx.x / s.blocks;
    const long long i = ((long long)(blockIdx.x % s.blocks) * kThreads + threadIdx.x) * L::N;
    const bool active = i < s.n;
    const long long at = active ? i : 0;   // idle lanes read voxel 0 and contribute zeros
    const T *gb = gy + b * s.channels * s.n + at, *xb = x + b * s.channels * s.n + at;
    T *ob = gx + b * s.channels * s.n + at;
    float mean[L::N], rstd[L::N], s1[L::N], s2[L::N];
#pragma unroll
    for (int e = 0; e < L::N; ++e) {
        mean[e] = stats[(b * 2 + 0) * s.n + at + e];
        rstd[e] = active ? stats[(b * 2 + 1) * s.n + at + e] : 0.f;
        s1[e] = s2[e] = 0.f;
    }
    float *mine = partial ? partial + ((long long)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6)) * s.channels * 2
                          : nullptr;
    L g, t;
    for (int c = 0; c < s.channels; ++c) {
        const float w = weight ? weight[c] : 1.f;
        g.load(gb + c * s.n);
        t.load(xb + c * s.n);
        float pw = 0.f, pb = 0.f;
#pragma unroll
        for (int e = 0; e < L::N; ++e) {
            const float gv = active ? g.v[e] : 0.f;
            const float xh = (t.v[e] - mean[e]) * rstd[e];
            s1[e] += gv * w;
            s2[e] += gv * w * xh;
            pw += gv * xh;
            pb += gv;
        }
        if (mine) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                pw += __shfl_down(pw, off, 64);
                pb += __shfl_down(pb, off, 64);
            }
            if ((threadIdx.x & 63) == 0) {
                mine[2 * c] = pw;
                mine[2 * c + 1] = pb;
            }
        }
    }
    if (!active) return;
    const float inv_c = 1.f / (float)s.channels;
    for (int c = 0; c < s.channels; ++c) {
        const float w = weight ? weight[c] : 1.f;
        g.load(gb + c * s.n);
        t.load(xb + c * s.n);
#pragma unroll
        for (int e = 0; e < L::N; ++e) {
            const float xh = (t.v[e] - mean[e]) * rstd[e];
            t.v[e] = rstd[e] * (g.v[e] * w - s1[e] * inv_c - xh * s2[e] * inv_c);
        }
        t.store(ob + c * s.n);
    }
}

}  // namespace chnorm
}  // namespace ndc
