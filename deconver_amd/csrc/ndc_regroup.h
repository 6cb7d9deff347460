// Regrouping of a grid by 2 x 2 (x 2) windows, the data movement of the network's 2-tap,
// stride-2 resampling convolutions (unet.py:36-60, 108-131 of the reference) once their
// arithmetic is a 1x1 projection:
//
//   to_channels:  out[r][k][d][h][w] = in[r][2d + kd][2h + kh][2w + kw]      k = (kd, kh, kw)
//   to_grid    :  out[r][2d + kd][2h + kh][2w + kw] = in[r][k][d][h][w] (+ bias[r % channels])
//
// for R rows (batch x channels) of a D x H x W grid (D = 1 and k = (kh, kw) in 2-D).  A thread
// moves 16 bytes of the fine grid: it splits them into even and odd columns (two 8-byte
// accesses to two planes of the coarse side) or interleaves them back.  Both sides are read and
// written in contiguous runs of at least half a row.  Device code only.
#pragma once
#include <hip/hip_runtime.h>

#include "ndc_common.h"

namespace ndc {
namespace regroup {

struct Shape {
    long long rows;
    int D, H, W;        // fine grid (even extents; D = 1 with depth2 = 0)
    int depth2;         // 1: windows of 2 along D as well
    int channels;       // rows % channels indexes the bias
};

// 16-bit elements: 8 per thread; x = (e0 e1) (e2 e3) (e4 e5) (e6 e7) as 32-bit words
__device__ inline void split16(const uint4 v, uint2 &even, uint2 &odd)
{
    even.x = __builtin_amdgcn_perm(v.y, v.x, 0x05040100u);
    odd.x = __builtin_amdgcn_perm(v.y, v.x, 0x07060302u);
    even.y = __builtin_amdgcn_perm(v.w, v.z, 0x05040100u);
    odd.y = __builtin_amdgcn_perm(v.w, v.z, 0x07060302u);
}

__device__ inline uint4 join16(const uint2 even, const uint2 odd)
{
    uint4 v;
    v.x = __builtin_amdgcn_perm(odd.x, even.x, 0x05040100u);
    v.y = __builtin_amdgcn_perm(odd.x, even.x, 0x07060302u);
    v.z = __builtin_amdgcn_perm(odd.y, even.y, 0x05040100u);
    v.w = __builtin_amdgcn_perm(odd.y, even.y, 0x07060302u);
    return v;
}

__device__ inline uint32_t add_bias16(uint32_t w, float b)
{
    return pack_bf16x2(bits_to_float(w << 16) + b, bits_to_float(w & 0xffff0000u) + b);
}

// ESZ = 2: W % 8 == 0; ESZ = 4: W % 4 == 0.  One thread per 16 bytes of the fine grid.
template <int ESZ, bool TO_CHANNELS>
__global__ void __launch_bounds__(256)
kernel(const void *src, void *dst, const float *bias, Shape s, long long nvec)
{
    constexpr int VN = 16 / ESZ;          // fine elements per thread
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= nvec) return;
    const int wv = s.W / VN;
    const int w = (int)(idx % wv) * VN;
    long long t = idx / wv;
    const int h = (int)(t % s.H);
    t /= s.H;
    const int d = (int)(t % s.D);
    const long long r = t / s.D;
    const int kd = s.depth2 ? (d & 1) : 0, kh = h & 1;
    const int Dc = s.depth2 ? s.D / 2 : 1, Hc = s.H / 2, Wc = s.W / 2;
    const int dc = s.depth2 ? d / 2 : 0, hc = h / 2;
    const int nk = s.depth2 ? 8 : 4;
    const long long plane = (long long)Dc * Hc * Wc;
    // coarse side: plane k = (kd, kh, kw) of row r, position (dc, hc, w / 2)
    const long long fine = ((r * s.D + d) * s.H + h) * (long long)s.W + w;
    const long long coarse = (r * nk + (kd * 2 + kh) * 2) * plane + ((long long)dc * Hc + hc) * Wc + w / 2;
    if (TO_CHANNELS) {
        const uint4 v = *reinterpret_cast<const uint4 *>((const char *)src + fine * ESZ);
        uint2 even, odd;
        if (ESZ == 2) {
            split16(v, even, odd);
        } else {
            even = make_uint2(v.x, v.z);
            odd = make_uint2(v.y, v.w);
        }
        *reinterpret_cast<uint2 *>((char *)dst + coarse * ESZ) = even;
        *reinterpret_cast<uint2 *>((char *)dst + (coarse + plane) * ESZ) = odd;
    } else {
        uint2 even = *reinterpret_cast<const uint2 *>((const char *)src + coarse * ESZ);
        uint2 odd = *reinterpret_cast<const uint2 *>((const char *)src + (coarse + plane) * ESZ);
        uint4 v;
        if (ESZ == 2) {
            v = join16(even, odd);
        } else {
            v = make_uint4(even.x, odd.x, even.y, odd.y);
        }
        if (bias) {
            const float b = bias[r % s.channels];
            if (ESZ == 2) {
                v.x = add_bias16(v.x, b);
                v.y = add_bias16(v.y, b);
                v.z = add_bias16(v.z, b);
                v.w = add_bias16(v.w, b);
            } else {
                v.x = float_to_bits(bits_to_float(v.x) + b);
                v.y = float_to_bits(bits_to_float(v.y) + b);
                v.z = float_to_bits(bits_to_float(v.z) + b);
                v.w = float_to_bits(bits_to_float(v.w) + b);
            }
        }
        *reinterpret_cast<uint4 *>((char *)dst + fine * ESZ) = v;
    }
}

}  // namespace regroup
}  // namespace ndc
