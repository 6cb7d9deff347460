// Row normalisation on the GPU: y = (x - mean(x)) / sqrt(var(x) + eps) over each row of a
// (rows, n) matrix, and its gradient.  On a channel-first tensor (B, C, *S) the rows are the
// B*C channel maps, i.e. this is InstanceNorm without affine parameters or running
// statistics -- the norm that sits between the NDC layers of the 3-D network, where a row is
// up to 128^3 elements long and there are as few as 128 rows.  A row is therefore cut into
// `nsplit` parts, one workgroup each, in two launches per direction:
//
//   reduce:  one partial result per (row, part)
//   apply :  every workgroup combines its row's nsplit partials (same order everywhere), then
//            transforms its part
//
//   forward : partial = (mean, sum of squared deviations from it) of the part, from sums of
//             x - pivot and (x - pivot)^2 with pivot = the mean of the row's first elements
//             (so the squares carry no cancellation); parts are combined pairwise-exactly
//             (Chan et al.); y = (x - mean) rstd;  stats[row] = (mean, rstd)
//   backward: partial = (sum gy, sum gy y);  gx = rstd (gy - mean(gy) - y mean(gy y)) [+ addend]
//
// The backward's optional addend is the gradient that reaches x by another way (the residual
// branch around a pre-norm block): summed here, it saves the separate pass that would add it.
//
// HBM traffic: forward 2 reads + 1 write of the tensor, backward 4 reads + 1 write.  Sums are
// float32 whatever the storage type.  Device code only (included by the HIP build).
#pragma once
#include <hip/hip_runtime.h>

#include "ndc_common.h"

namespace ndc {
namespace rownorm {

static constexpr int kThreads = 256;
static constexpr int kMaxSplit = 64;

template <typename T> struct Vec;   // 16 bytes of T
template <> struct Vec<float> {
    static constexpr int N = 4;
    float4 v;
    __device__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
    __device__ void set(int i, float f) { (i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w) = f; }
};
template <> struct Vec<bf16_t> {
    static constexpr int N = 8;
    uint4 v;
    __device__ uint32_t word(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
    __device__ float get(int i) const
    {
        const uint32_t w = word(i >> 1);
        return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
    }
    __device__ void set_pair(int p, float lo, float hi)
    {
        (p == 0 ? v.x : p == 1 ? v.y : p == 2 ? v.z : v.w) = pack_bf16x2(lo, hi);
    }
};

// (sum over the workgroup of a, of b) in every thread; fixed association
__device__ inline void block_sum2(float &a, float &b, float (*buf)[2])
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_down(a, off, 64);
        b += __shfl_down(b, off, 64);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        buf[wave][0] = a;
        buf[wave][1] = b;
    }
    __syncthreads();
    a = (buf[0][0] + buf[1][0]) + (buf[2][0] + buf[3][0]);
    b = (buf[0][1] + buf[1][1]) + (buf[2][1] + buf[3][1]);
    __syncthreads();
}

// the row's totals from its nsplit partials, in every thread
__device__ inline void row_totals(const float2 *partial, int nsplit, float &s1, float &s2, float (*buf)[2])
{
    if (threadIdx.x < 64) {
        float a = 0.f, b = 0.f;
        if ((int)threadIdx.x < nsplit) {
            const float2 p = partial[threadIdx.x];
            a = p.x;
            b = p.y;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            a += __shfl_down(a, off, 64);
            b += __shfl_down(b, off, 64);
        }
        if (threadIdx.x == 0) {
            buf[0][0] = a;
            buf[0][1] = b;
        }
    }
    __syncthreads();
    s1 = buf[0][0];
    s2 = buf[0][1];
}

struct Split {
    long long n;        // row length, elements
    long long chunk;    // elements per part (a multiple of the vector width)
    int nsplit;
};

template <typename T, bool BWD, bool VEC>
__global__ void __launch_bounds__(kThreads)
reduce_kernel(const T *a, const T *b, float2 *partial, Split sp)
{
    __shared__ float buf[4][2];
    const long long row = blockIdx.x / sp.nsplit;
    const int part = blockIdx.x % sp.nsplit;
    const T *ar = a + row * sp.n, *br = BWD ? b + row * sp.n : nullptr;
    const long long lo = part * sp.chunk, hi = lo + sp.chunk < sp.n ? lo + sp.chunk : sp.n;
    float pivot = 0.f;
    if (!BWD) {
        // the mean of the row's first elements (one access per thread), the same in every part
        float head = 0.f, unused = 0.f;
        long long cnt;
        if constexpr (VEC) {
            typedef Vec<T> V;
            const long long nv = sp.n / V::N;
            cnt = (nv < kThreads ? nv : kThreads) * V::N;
            if ((long long)threadIdx.x < nv) {
                const V x = reinterpret_cast<const V *>(ar)[threadIdx.x];
#pragma unroll
                for (int e = 0; e < V::N; ++e) head += x.get(e);
            }
        } else {
            cnt = sp.n < kThreads ? sp.n : kThreads;
            if ((long long)threadIdx.x < sp.n) head = Elem<T>::load(ar + threadIdx.x);
        }
        block_sum2(head, unused, buf);
        pivot = head / (float)cnt;
    }
    float s1 = 0.f, s2 = 0.f;
    if constexpr (VEC) {
        typedef Vec<T> V;
        const long long v0 = lo / V::N, v1 = hi / V::N;
        const V *av = reinterpret_cast<const V *>(ar), *bv = reinterpret_cast<const V *>(br);
        float t1[4] = {0.f, 0.f, 0.f, 0.f}, t2[4] = {0.f, 0.f, 0.f, 0.f};
        long long i = v0 + threadIdx.x;
        for (; i + 3 * kThreads < v1; i += 4 * kThreads) {
            V x[4], y[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                x[u] = av[i + u * kThreads];
                if (BWD) y[u] = bv[i + u * kThreads];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < V::N; ++e) {
                    const float f = x[u].get(e) - pivot;
                    t1[u] += f;
                    t2[u] += f * (BWD ? y[u].get(e) : f);
                }
        }
        for (; i < v1; i += kThreads) {
            const V x = av[i];
            V y;
            if (BWD) y = bv[i];
#pragma unroll
            for (int e = 0; e < V::N; ++e) {
                const float f = x.get(e) - pivot;
                t1[0] += f;
                t2[0] += f * (BWD ? y.get(e) : f);
            }
        }
        s1 = (t1[0] + t1[1]) + (t1[2] + t1[3]);
        s2 = (t2[0] + t2[1]) + (t2[2] + t2[3]);
    } else {
        for (long long i = lo + threadIdx.x; i < hi; i += kThreads) {
            const float f = Elem<T>::load(ar + i) - pivot;
            s1 += f;
            s2 += f * (BWD ? Elem<T>::load(br + i) : f);
        }
    }
    block_sum2(s1, s2, buf);
    if (threadIdx.x == 0) {
        if (!BWD) {
            const float inv = 1.f / (float)(hi - lo);
            partial[blockIdx.x] = make_float2(pivot + s1 * inv, s2 - s1 * s1 * inv);
        } else {
            partial[blockIdx.x] = make_float2(s1, s2);
        }
    }
}

// partial[row][part] = the sum of the part: the bias gradient of a projection without activation
// is the sum of its output gradient over batch, parts and voxels (1 U e read).
template <typename T, bool VEC>
__global__ void __launch_bounds__(kThreads)
row_sums_kernel(const T *a, float *partial, Split sp)
{
    __shared__ float buf[4][2];
    const long long row = blockIdx.x / sp.nsplit;
    const int part = blockIdx.x % sp.nsplit;
    const T *ar = a + row * sp.n;
    const long long lo = part * sp.chunk, hi = lo + sp.chunk < sp.n ? lo + sp.chunk : sp.n;
    float s = 0.f, unused = 0.f;
    if constexpr (VEC) {
        typedef Vec<T> V;
        const long long v0 = lo / V::N, v1 = hi / V::N;
        const V *av = reinterpret_cast<const V *>(ar);
        float t[4] = {0.f, 0.f, 0.f, 0.f};
        long long i = v0 + threadIdx.x;
        for (; i + 3 * kThreads < v1; i += 4 * kThreads) {
            V x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = av[i + u * kThreads];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < V::N; ++e) t[u] += x[u].get(e);
        }
        for (; i < v1; i += kThreads) {
            const V x = av[i];
#pragma unroll
            for (int e = 0; e < V::N; ++e) t[0] += x.get(e);
        }
        s = (t[0] + t[1]) + (t[2] + t[3]);
    } else {
        for (long long i = lo + threadIdx.x; i < hi; i += kThreads) s += Elem<T>::load(ar + i);
    }
    block_sum2(s, unused, buf);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

template <typename T, bool BWD, bool VEC, bool ADD = false>
__global__ void __launch_bounds__(kThreads)
apply_kernel(const T *a, const T *b, const T *addend, const float2 *partial, float2 *stats, T *out, Split sp,
             float eps)
{
    __shared__ float buf[4][2];
    const long long row = blockIdx.x / sp.nsplit;
    const int part = blockIdx.x % sp.nsplit;
    const T *ar = a + row * sp.n, *br = BWD ? b + row * sp.n : nullptr;
    const T *dr = ADD ? addend + row * sp.n : nullptr;
    T *orow = out + row * sp.n;
    const long long lo = part * sp.chunk, hi = lo + sp.chunk < sp.n ? lo + sp.chunk : sp.n;
    const float inv_n = 1.f / (float)sp.n;
    // forward: out = (x - c0) * c1;  backward: out = gy * c1 + y * c2 + c0
    float c0, c1, c2 = 0.f;
    if (BWD) {
        float s1, s2;
        row_totals(partial + row * sp.nsplit, sp.nsplit, s1, s2, buf);
        const float rstd = stats[row].y;
        c1 = rstd;
        c0 = -rstd * s1 * inv_n;
        c2 = -rstd * s2 * inv_n;
    } else {
        // (count, mean, squared deviations) of the parts merged in order, by every thread
        float cnt = 0.f, mean = 0.f, m2 = 0.f;
        for (int p = 0; p < sp.nsplit; ++p) {
            const float2 q = partial[row * sp.nsplit + p];
            const long long plo = p * sp.chunk, phi = plo + sp.chunk < sp.n ? plo + sp.chunk : sp.n;
            const float np = (float)(phi - plo), tot = cnt + np, delta = q.x - mean;
            mean += delta * (np / tot);
            m2 += q.y + delta * delta * (cnt * np / tot);
            cnt = tot;
        }
        float var = m2 * inv_n;
        var = var > 0.f ? var : 0.f;
        const float rstd = 1.f / sqrtf(var + eps);
        c1 = rstd;
        c0 = mean;
        if (part == 0 && threadIdx.x == 0) stats[row] = make_float2(mean, rstd);
    }
    if constexpr (VEC) {
        typedef Vec<T> V;
        const long long v0 = lo / V::N, v1 = hi / V::N;
        const V *av = reinterpret_cast<const V *>(ar), *bv = reinterpret_cast<const V *>(br);
        const V *dv = reinterpret_cast<const V *>(dr);
        V *ov = reinterpret_cast<V *>(orow);
        auto one = [&](const V &x, const V &y, const V &d) {
            V r;
            float v[V::N];
#pragma unroll
            for (int e = 0; e < V::N; ++e) {
                v[e] = BWD ? x.get(e) * c1 + c0 + y.get(e) * c2 : (x.get(e) - c0) * c1;
                if (ADD) v[e] += d.get(e);
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
            V x[4], y[4], d[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                x[u] = av[i + u * kThreads];
                if (BWD) y[u] = bv[i + u * kThreads];
                if (ADD) d[u] = dv[i + u * kThreads];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) ov[i + u * kThreads] = one(x[u], y[u], d[u]);
        }
        for (; i < v1; i += kThreads) {
            const V x = av[i];
            V y, d;
            if (BWD) y = bv[i];
            if (ADD) d = dv[i];
            ov[i] = one(x, y, d);
        }
    } else {
        for (long long i = lo + threadIdx.x; i < hi; i += kThreads) {
            const float v = Elem<T>::load(ar + i);
            float f = BWD ? v * c1 + c0 + Elem<T>::load(br + i) * c2 : (v - c0) * c1;
            if (ADD) f += Elem<T>::load(dr + i);
            Elem<T>::store(orow + i, f);
        }
    }
}

}  // namespace rownorm
}  // namespace ndc
