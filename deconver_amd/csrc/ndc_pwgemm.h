// The 1x1 projections of a Deconver block as a streaming GEMM on channel-first bf16 tensors,
//
//   y[b][co][v] = act( sum_ci W[co][ci] * x[b][ci][v] + bias[co] ) + residual[b][co][v],
//
// (layers/linear.py:53-58 of the reference: nn.Conv1d with kernel size 1; with the activation
// and the residual sum of the block that calls it, deconver.py:41-46, 60-64, layers/mlp.py:40-63).
//
// These products are skinny: 64-512 channels on either side, millions of voxels, so every
// element of x is read once and every element of y written once and the arithmetic
// (2 * cin * cout flops per voxel) needs a tenth of the matrix units while the tensors stream:
// the kernel is built for HBM bandwidth, not for matrix throughput.  One wavefront owns 64
// consecutive voxels of one sample at a time and produces ALL output channels for them:
//
//   * x is read straight from global memory into the B operand of
//     v_mfma_f32_32x32x16_bf16.  That operand wants, per lane, 8 consecutive input channels of
//     ONE voxel, while memory has voxels contiguous.  Lane (n, kb) of 64 = 32 x 2 therefore
//     loads the 4-byte word (voxel 2n, voxel 2n+1) of the 8 channels 16 s + 8 kb + 0..7 of
//     k-step s (half a wavefront covers 128 contiguous bytes of one channel row per load) and
//     splits the 8 words with 8 v_perm_b32 into the fragments of two 32-voxel tiles: tile 0
//     holds the even voxels, tile 1 the odd ones.  No LDS, no second read of x.
//   * W comes packed in fragment order (pack_kernel: the 16 bytes lane l needs for output
//     tile c and k-step s lie at ((c * S + s) * 64 + l) * 16), is copied into LDS once per
//     workgroup and read from there with one 16-byte access per matrix instruction, without
//     bank conflicts.  Workgroups are persistent: wavefront g of G takes tiles g, g + G, ...
//   * The accumulators of tile 0 and tile 1 hold, in the same lane and register, the two
//     voxels of one output word, so the epilogue (bias, activation, residual, optional copy
//     of the product before bias for the activation's gradient) works on words and every
//     store is again 128 contiguous bytes per half wavefront.
//
// Whatever the instruction's internal order of the 16 k-values is, both operands are filled by
// the same rule (lane half kb, element e <-> channel 16 s + 8 kb + e), so the products pair up.
// Two kernels: gemm_kernel holds the fragments of up to 256 input channels whole and walks the
// output tiles one after the other (any number of output channels; also the modes that multiply
// the product by an activation's derivative and sum the result per channel); gemm_kernel_deep
// takes more input channels in chunks of 64 with the accumulators of all (at most four) output
// tiles kept (these are the projections back from a widened tensor: bias and residual only, no
// activation, nothing kept).  Device code only; float32 accumulation; the output is rounded to bf16 once.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ndc_common.h"
#include "ndc_epilogue.h"

namespace ndc {
namespace pwgemm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

static const int kTileVoxels = 64;       // voxels a wavefront owns at a time
static const int kMaxParts = 4096;       // wavefronts of a launch (rows of Params::gpart) at most
// Epilogue modes beyond epilogue::kNone / kRelu / kGelu: the product times the activation's
// derivative at (aux + bias), aux read through Params::res -- the input gradient of a
// projection whose INPUT was act(aux + bias) (the MLP's second projection, layers/mlp.py:40-63)
enum { kReluGrad = 3, kGeluGrad = 4 };
// ... and kMasked: y = (W x + bias + residual) where mask > 0, else 0 -- an input gradient taken
// through the rectifier that made the projection's input (mask: that rectifier's output), with
// another gradient of the same tensor accumulated on the way (residual)
enum { kMasked = 5 };

struct Params {
    const uint16_t *x;       // (B, cin, n) bf16
    const uint16_t *wfrag;   // cout/32 * cin/16 fragments of 64 lanes x 8 bf16 (pack_kernel)
    const float *bias;       // cout values or null
    const uint16_t *res;     // (B, cout, n) or null
    uint16_t *y;             // (B, cout, n)
    uint16_t *zkeep;         // (B, cout, n) or null: the product before bias and activation
    float *gpart;            // gradient modes: (gridDim.x * waves, cout) sums of y per wavefront, or null
    const uint16_t *mask;    // kMasked: (B, cout, n)
    long long n;             // voxels per sample, a multiple of 64
    int tiles;               // B * n / 64
    int tiles_per_sample;
    int cout;                // a multiple of 32
};

// W (cout x cin, row-major, float32 or bf16; or its transpose stored as cin x cout when
// TRANSPOSED) -> fragment order.  One thread per (fragment, lane); tiny.
template <typename TW, bool TRANSPOSED>
__global__ void pack_kernel(const TW *w, uint16_t *wfrag, int cout, int cin)
{
    const int S = cin / 16;
    const long long id = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (long long)(cout / 32) * S * 64) return;
    const int lane = (int)(id & 63);
    const long long frag = id >> 6;
    const int s = (int)(frag % S), c = (int)(frag / S);
    const int row = 32 * c + (lane & 31), k0 = 16 * s + 8 * (lane >> 5);
    uint32_t out[4];
#pragma unroll
    for (int pr = 0; pr < 4; ++pr) {
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = k0 + 2 * pr + h;
            const long long at = TRANSPOSED ? (long long)k * cout + row : (long long)row * cin + k;
            v[h] = Elem<TW>::load(w + at);
        }
        out[pr] = pack_bf16x2(v[0], v[1]);
    }
    u32x4 o = {out[0], out[1], out[2], out[3]};
    reinterpret_cast<u32x4 *>(wfrag)[id] = o;
}

__device__ inline float lo_bf16(uint32_t w) { return __uint_as_float(w << 16); }
__device__ inline float hi_bf16(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Addresses are a wavefront-uniform pointer (scalar registers) plus a 32-bit lane offset in
// words, so that no 64-bit address lives in vector registers: 2 * n + 32 words must fit 32 bits.
__device__ inline const uint32_t *words(const uint16_t *p) { return reinterpret_cast<const uint32_t *>(p); }
__device__ inline uint32_t *words(uint16_t *p) { return reinterpret_cast<uint32_t *>(p); }

// the 8 words (voxel 2n, voxel 2n + 1) of every k-step of a tile; xw: lane offset 4 kb n + n32
template <int S>
__device__ inline void request_x(const Params &p, int tile, int cin, uint32_t xw, uint32_t (&raw)[S][8], int k0 = 0)
{
    // (the quotient comes out of vector arithmetic; as a scalar again it keeps the pointers scalar)
    const int b = __builtin_amdgcn_readfirstlane(tile / p.tiles_per_sample);
    const uint16_t *xb = p.x + (long long)b * cin * p.n + (long long)(tile - b * p.tiles_per_sample) * kTileVoxels;
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) raw[s][e] = words(xb + (long long)(k0 + 16 * s + e) * p.n)[xw];
}

// ... into the fragments of the even-voxel tile and the odd-voxel tile
template <int S>
__device__ inline void split_x(const uint32_t (&raw)[S][8], bf16x8 (&xf)[S][2])
{
#pragma unroll
    for (int s = 0; s < S; ++s) {
        u32x4 even, odd;
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
            even[pr] = __builtin_amdgcn_perm(raw[s][2 * pr + 1], raw[s][2 * pr], 0x05040100u);
            odd[pr] = __builtin_amdgcn_perm(raw[s][2 * pr + 1], raw[s][2 * pr], 0x07060302u);
        }
        xf[s][0] = __builtin_bit_cast(bf16x8, even);
        xf[s][1] = __builtin_bit_cast(bf16x8, odd);
    }
}

// The epilogue of one 32-channel output tile of gemm_kernel_deep (bias and residual only).  Register j of a lane holds output
// row 8 * (j / 4) + 4 * kb + j % 4, column n32, of the even-voxel tile (acc0) and the odd-voxel
// tile (acc1): one output word.  rw: the residual words, requested by the caller.
template <bool RES, bool MASK>
__device__ inline void finish_tile(const Params &p, const f32x16 &acc0, const f32x16 &acc1, const uint32_t (&rw)[16],
                                   const uint32_t (&mw)[16], const float *bl, int c, long long at0, uint32_t yw, int kb)
{
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 t4 = *reinterpret_cast<const float4 *>(bl + 32 * c + 8 * q + 4 * kb);
        const float bq[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int j = 4 * q + jj;
            const long long at = at0 + (long long)(8 * q + jj) * p.n;
            const float z0 = acc0[j], z1 = acc1[j];
            float y0 = z0 + bq[jj], y1 = z1 + bq[jj];
            if constexpr (RES) y0 += lo_bf16(rw[j]), y1 += hi_bf16(rw[j]);
            if constexpr (MASK) y0 = lo_bf16(mw[j]) > 0.f ? y0 : 0.f, y1 = hi_bf16(mw[j]) > 0.f ? y1 : 0.f;
            words(p.y + at)[yw] = pack_bf16x2(y0, y1);
        }
    }
}

template <int CIN, int ACT, bool RES, int THREADS>
__global__ void __launch_bounds__(THREADS) gemm_kernel(Params p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int S = CIN / 16;
    constexpr int WAVES = THREADS / 64;
    u32x4 *wl = reinterpret_cast<u32x4 *>(smem);
    const int CT = p.cout / 32;
    // the bias sits in LDS behind the weights (zeros without one): a global load among the
    // epilogue's stores would have to wait for all of them (one counter for loads and stores)
    float *bl = reinterpret_cast<float *>(smem + (size_t)CT * S * 64 * 16);
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(p.wfrag);
        const int chunks = CT * S * 64;
        for (int i = threadIdx.x; i < chunks; i += THREADS) wl[i] = src[i];
        for (int i = threadIdx.x; i < p.cout; i += THREADS) bl[i] = p.bias ? p.bias[i] : 0.f;
    }
    constexpr bool GRAD = ACT == kReluGrad || ACT == kGeluGrad;
    static_assert(!GRAD || RES, "the gradient modes read aux through the residual pointer");
    // gradient modes: every wavefront sums y per output channel in a row of its own (LDS)
    float *gs = bl + p.cout + (threadIdx.x >> 6) * p.cout;
    if constexpr (GRAD)
        for (int i = threadIdx.x; i < WAVES * p.cout; i += THREADS) bl[p.cout + i] = 0.f;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // tile indices stay scalar
    const int n32 = lane & 31, kb = lane >> 5;
    const uint32_t xw = (uint32_t)(4 * kb) * (uint32_t)p.n + n32;   // lane offsets in words:
    const uint32_t yw = (uint32_t)(2 * kb) * (uint32_t)p.n + n32;   // 8 kb rows of x, 4 kb rows of y
    const int nwaves = (int)gridDim.x * WAVES;
    // (Requesting a tile's words one tile ahead was measured, with 64 and 128 input channels:
    // no gain at 64, a loss at 128 -- the resident wavefronts already cover the latency.)
    for (int tile = (int)blockIdx.x * WAVES + wave; tile < p.tiles; tile += nwaves) {
        const int b = __builtin_amdgcn_readfirstlane(tile / p.tiles_per_sample);
        bf16x8 xf[S][2];
        {
            uint32_t raw[S][8];
            request_x<S>(p, tile, CIN, xw, raw);
            split_x<S>(raw, xf);
        }
        // ---- one 32-channel output tile after the other.  Register j of a lane holds output
        // row 8 * (j / 4) + 4 * kb + j % 4, column n32.  The residual words of a tile are
        // requested before its matrix instructions, so that they arrive behind them.
        const long long out0 = (long long)b * p.cout * p.n + (long long)(tile - b * p.tiles_per_sample) * kTileVoxels;
#pragma unroll 1
        for (int c = 0; c < CT; ++c) {
            const long long at0 = out0 + (long long)(32 * c) * p.n;
            uint32_t rw[16], mw[16];
            if constexpr (RES) {
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    rw[j] = words(p.res + at0 + (long long)(8 * (j / 4) + j % 4) * p.n)[yw];
            }
            if constexpr (ACT == kMasked) {
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    mw[j] = words(p.mask + at0 + (long long)(8 * (j / 4) + j % 4) * p.n)[yw];
            }
            f32x16 acc0 = {}, acc1 = {};
            const u32x4 *wt = wl + (c * S) * 64 + lane;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const bf16x8 wf = __builtin_bit_cast(bf16x8, wt[s * 64]);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[s][0], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[s][1], acc1, 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 t4 = *reinterpret_cast<const float4 *>(bl + 32 * c + 8 * q + 4 * kb);
                const float bq[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int j = 4 * q + jj;
                    const long long at = at0 + (long long)(8 * q + jj) * p.n;
                    const float z0 = acc0[j], z1 = acc1[j];
                    float y0, y1;
                    if constexpr (GRAD) {
                        constexpr int A = ACT == kGeluGrad ? epilogue::kGelu : epilogue::kRelu;
                        y0 = z0 * epilogue::act_grad<A>(lo_bf16(rw[j]) + bq[jj]);
                        y1 = z1 * epilogue::act_grad<A>(hi_bf16(rw[j]) + bq[jj]);
                        // the channel's sum over the tile's 64 voxels: the 32 lanes of this half
                        float t = y0 + y1;
#pragma unroll
                        for (int m = 1; m < 32; m <<= 1) t += __shfl_xor(t, m);
                        if (p.gpart && n32 == 0) gs[32 * c + 8 * q + 4 * kb + jj] += t;
                    } else if constexpr (ACT == kMasked) {
                        y0 = z0 + bq[jj], y1 = z1 + bq[jj];
                        if constexpr (RES) y0 += lo_bf16(rw[j]), y1 += hi_bf16(rw[j]);
                        y0 = lo_bf16(mw[j]) > 0.f ? y0 : 0.f, y1 = hi_bf16(mw[j]) > 0.f ? y1 : 0.f;
                    } else {
                        if constexpr (ACT != epilogue::kNone) {   // (kept only for an activation's gradient)
                            if (p.zkeep) words(p.zkeep + at)[yw] = pack_bf16x2(z0, z1);
                        }
                        y0 = epilogue::act_fwd<ACT>(z0 + bq[jj]), y1 = epilogue::act_fwd<ACT>(z1 + bq[jj]);
                        if constexpr (RES) y0 += lo_bf16(rw[j]), y1 += hi_bf16(rw[j]);
                    }
                    words(p.y + at)[yw] = pack_bf16x2(y0, y1);
                }
            }
        }
    }
    if constexpr (GRAD) {
        // (only this wavefront touched its row; lanes 0 and 32 wrote it, all lanes read it)
        if (p.gpart) {
            __builtin_amdgcn_wave_barrier();
            const int g = (int)blockIdx.x * WAVES + wave;
            float *row = p.gpart + (long long)g * p.cout;
            for (int i = lane; i < p.cout; i += 64) row[i] = gs[i];
            // rows beyond the launch's wavefronts read zero (written here, not by a memset, so
            // that the call can be recorded into a graph)
            for (int r = g + nwaves; r < kMaxParts; r += nwaves)
                for (int i = lane; i < p.cout; i += 64) p.gpart[(long long)r * p.cout + i] = 0.f;
        }
    }
}

// Many input channels, at most 128 output channels (the projections back from the widened
// tensors: 512 -> 128): the accumulators of ALL CT output tiles stay in registers while the
// input channels go by in chunks of 64, so that x is still read once.  cin: a multiple of 64.
template <int CT, bool RES, bool MASK, int THREADS>
__global__ void __launch_bounds__(THREADS) gemm_kernel_deep(Params p, int cin)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int WAVES = THREADS / 64;
    constexpr int SC = 4;                    // k-steps per chunk of 64 input channels
    const int S = cin / 16, chunks_k = cin / 64;
    u32x4 *wl = reinterpret_cast<u32x4 *>(smem);
    float *bl = reinterpret_cast<float *>(smem + (size_t)CT * S * 64 * 16);
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(p.wfrag);
        const int chunks = CT * S * 64;
        for (int i = threadIdx.x; i < chunks; i += THREADS) wl[i] = src[i];
        for (int i = threadIdx.x; i < 32 * CT; i += THREADS) bl[i] = p.bias ? p.bias[i] : 0.f;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n32 = lane & 31, kb = lane >> 5;
    const uint32_t xw = (uint32_t)(4 * kb) * (uint32_t)p.n + n32;
    const uint32_t yw = (uint32_t)(2 * kb) * (uint32_t)p.n + n32;
    const int nwaves = (int)gridDim.x * WAVES;
    for (int tile = (int)blockIdx.x * WAVES + wave; tile < p.tiles; tile += nwaves) {
        const int b = __builtin_amdgcn_readfirstlane(tile / p.tiles_per_sample);
        f32x16 acc[CT][2];
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[c][0] = f32x16{}, acc[c][1] = f32x16{};
#pragma unroll 1
        for (int kc = 0; kc < chunks_k; ++kc) {
            uint32_t raw[SC][8];
            request_x<SC>(p, tile, cin, xw, raw, 64 * kc);
            bf16x8 xf[SC][2];
            split_x<SC>(raw, xf);
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                const u32x4 *wt = wl + (c * S + kc * SC) * 64 + lane;
#pragma unroll
                for (int s = 0; s < SC; ++s) {
                    const bf16x8 wf = __builtin_bit_cast(bf16x8, wt[s * 64]);
                    acc[c][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[s][0], acc[c][0], 0, 0, 0);
                    acc[c][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[s][1], acc[c][1], 0, 0, 0);
                }
            }
        }
        const long long out0 = (long long)b * p.cout * p.n + (long long)(tile - b * p.tiles_per_sample) * kTileVoxels;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const long long at0 = out0 + (long long)(32 * c) * p.n;
            uint32_t rw[16], mw[16];
            if constexpr (RES) {
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    rw[j] = words(p.res + at0 + (long long)(8 * (j / 4) + j % 4) * p.n)[yw];
            }
            if constexpr (MASK) {
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    mw[j] = words(p.mask + at0 + (long long)(8 * (j / 4) + j % 4) * p.n)[yw];
            }
            finish_tile<RES, MASK>(p, acc[c][0], acc[c][1], rw, mw, bl, c, at0, yw, kb);
        }
    }
}

}  // namespace pwgemm
}  // namespace ndc
