// HIP (gfx950) build of the NDC C ABI: launch primitives + the shared host logic.
#include <hip/hip_runtime.h>

#include <atomic>

#include "ndc_common.h"
#include "ndc_exec.h"
#include "ndc_rownorm.h"
#include "ndc_epilogue.h"
#include "ndc_regroup.h"
#include "ndc_chnorm.h"
#include "ndc_pwgemm.h"

#define NDC_LAMBDA __host__ __device__

namespace ndc {

template <class F>
__global__ void __launch_bounds__(256) elementwise_kernel(long long n, F f)
{
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += stride)
        f(idx);
}

template <class F>
__global__ void __launch_bounds__(256) block_reduce_kernel(float *out, F partial)
{
    __shared__ float buf[256];
    const int tid = threadIdx.x;
    buf[tid] = partial((int)blockIdx.x, tid, 256);
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (tid < s) buf[tid] += buf[tid + s];
        __syncthreads();
    }
    if (tid == 0) out[blockIdx.x] = buf[0];
}

// put(o, sum over p < nparts of term(o, p)) for o < nout.  A workgroup sums 32 outputs:
// thread (o, j), j < 8, adds the terms p = j, j + 8, ... in order, then thread (o, 0) adds the
// eight partial sums in order -- a fixed association, so results are reproducible.  Threads
// with consecutive o are neighbours, so a `term` that is contiguous in o reads coalesced.
template <class P, class F>
__global__ void __launch_bounds__(256) strided_sum_kernel(int nout, int nparts, P put, F term)
{
    __shared__ float buf[8][33];
    const int ox = threadIdx.x & 31, j = threadIdx.x >> 5;
    const int o = (int)blockIdx.x * 32 + ox;
    float acc = 0.f;
    if (o < nout)
        for (int p = j; p < nparts; p += 8) acc += term(o, p);
    buf[j][ox] = acc;
    __syncthreads();
    if (j == 0 && o < nout) {
        float total = 0.f;
#pragma unroll
        for (int k = 0; k < 8; ++k) total += buf[k][ox];
        put(o, total);
    }
}

// Batched matrix transposition dst[b][k][r] = src[b][r][k] (R rows, K columns per batch entry)
// of 16-bit elements, two at a time: a workgroup moves a 64 x 64 tile through LDS, reading
// 32-bit words along K and writing 32-bit words along R (R, K even, both pointers 4-byte
// aligned).  The copy between the channels-last layout (B, S, C) and the channel-first layout
// (B, C, S) the update kernels read is this transposition with (R, K) = (S, C) or (C, S).
__global__ void __launch_bounds__(256)
transpose_pairs_kernel(const uint32_t *src, uint32_t *dst, long long R, long long K, long long tiles_r,
                       long long tiles_k)
{
    __shared__ uint16_t tile[64][66];
    long long blk = blockIdx.x;
    const long long tk = blk % tiles_k;
    blk /= tiles_k;
    const long long tr = blk % tiles_r, b = blk / tiles_r;
    const long long row0 = tr * 64, col0 = tk * 64;
    const uint32_t *s = src + b * (R * K / 2);
    uint32_t *d = dst + b * (R * K / 2);
    const int w = threadIdx.x & 31, q = threadIdx.x >> 5;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int r = q + 8 * it;
        uint32_t v = 0u;
        if (row0 + r < R && col0 + 2 * w < K) v = s[((row0 + r) * K + col0) / 2 + w];
        *reinterpret_cast<uint32_t *>(&tile[r][2 * w]) = v;
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int k = q + 8 * it;
        if (col0 + k < K && row0 + 2 * w < R)
            d[((col0 + k) * R + row0) / 2 + w] = (uint32_t)tile[2 * w][k] | ((uint32_t)tile[2 * w + 1][k] << 16);
    }
}

// The same for elements of ESZ bytes (2 or 4), one at a time: any R, K and alignment.
template <typename E>
__global__ void __launch_bounds__(256)
transpose_kernel(const E *src, E *dst, long long R, long long K, long long tiles_r, long long tiles_k)
{
    __shared__ E tile[32][33];
    long long blk = blockIdx.x;
    const long long tk = blk % tiles_k;
    blk /= tiles_k;
    const long long tr = blk % tiles_r, b = blk / tiles_r;
    const long long row0 = tr * 32, col0 = tk * 32;
    const E *s = src + b * R * K;
    E *d = dst + b * R * K;
    const int w = threadIdx.x & 31, q = threadIdx.x >> 5;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int r = q + 8 * it;
        tile[r][w] = (row0 + r < R && col0 + w < K) ? s[(row0 + r) * K + col0 + w] : (E)0;
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int k = q + 8 * it;
        if (col0 + k < K && row0 + w < R) d[(col0 + k) * R + row0 + w] = tile[w][k];
    }
}

// One workgroup of an LDS-tiled kernel.  512 threads at most, so up to 256 VGPRs per lane.
template <class Kernel>
__global__ void __launch_bounds__(512) block_kernel_entry(typename Kernel::Params p)
{
    extern __shared__ __attribute__((aligned(16))) float ndc_lds[];
    DeviceExec<typename Kernel::State> ex;
    ex.lds = ndc_lds;
    ex.tid = threadIdx.x;
    ex.nthreads = blockDim.x;
    Kernel::run(ex, p, (int)blockIdx.x);
}

// The same for a kernel that declares `kWavesPerSimd = 4`: its LDS footprint lets four
// workgroups share a CU, so the register allocator is held to the 128 VGPRs that four
// wavefronts per SIMD leave each lane.
template <class Kernel>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
block_kernel_entry_w4(typename Kernel::Params p)
{
    extern __shared__ __attribute__((aligned(16))) float ndc_lds[];
    DeviceExec<typename Kernel::State> ex;
    ex.lds = ndc_lds;
    ex.tid = threadIdx.x;
    ex.nthreads = blockDim.x;
    Kernel::run(ex, p, (int)blockIdx.x);
}

template <class K, class = void> struct WavesWanted {
    static constexpr int value = 0;
};
template <class K> struct WavesWanted<K, decltype((void)K::kWavesPerSimd)> {
    static constexpr int value = K::kWavesPerSimd;
};

// Event stopwatch on one stream: mark() after each stage, finish() synchronises and
// reports the stage durations in milliseconds.
struct HipTimer {
    static const int kMax = 8;
    hipEvent_t ev[kMax + 1];
    int n = 0;
    bool on;
    hipStream_t stream;
    HipTimer(bool enable, void *s) : on(enable), stream((hipStream_t)s)
    {
        if (!on) return;
        for (int i = 0; i <= kMax; ++i) (void)hipEventCreate(&ev[i]);
        (void)hipEventRecord(ev[0], stream);
    }
    void mark()
    {
        if (on && n < kMax) (void)hipEventRecord(ev[++n], stream);
    }
    void finish(float *ms, int count)
    {
        if (!on) return;
        (void)hipEventSynchronize(ev[n]);
        for (int i = 0; i < count; ++i) {
            ms[i] = 0.f;
            if (i < n) (void)hipEventElapsedTime(&ms[i], ev[i], ev[i + 1]);
        }
        for (int i = 0; i <= kMax; ++i) (void)hipEventDestroy(ev[i]);
        on = false;
    }
    ~HipTimer() { if (on) for (int i = 0; i <= kMax; ++i) (void)hipEventDestroy(ev[i]); }
};

struct Backend {
    static constexpr bool is_device = true;
    typedef HipTimer Timer;

    template <class Kernel>
    static int block_kernel(const typename Kernel::Params &p, int nblocks, int nthreads,
                            int lds_floats, void *stream)
    {
        if (nblocks <= 0) return 0;
        const size_t bytes = (size_t)lds_floats * sizeof(float);
        void (*entry)(typename Kernel::Params) = block_kernel_entry<Kernel>;
        if constexpr (WavesWanted<Kernel>::value == 4) entry = block_kernel_entry_w4<Kernel>;
        if (bytes > 64 * 1024) {
            // more dynamic LDS than the default cap: raise it for this kernel (idempotent)
            if (hipFuncSetAttribute((const void *)entry, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)bytes) != hipSuccess)
                return -5;
        }
        hipLaunchKernelGGL(entry, dim3((unsigned)nblocks), dim3((unsigned)nthreads), bytes,
                           (hipStream_t)stream, p);
        return check();
    }

    static int check()
    {
        return hipGetLastError() == hipSuccess ? 0 : -5;
    }

    template <class F> static int elementwise(long long n, void *stream, F f)
    {
        if (n <= 0) return 0;
        long long blocks = (n + 255) / 256;
        if (blocks > (1LL << 20)) blocks = 1LL << 20;  // grid-stride beyond that
        hipLaunchKernelGGL(elementwise_kernel<F>, dim3((unsigned)blocks), dim3(256), 0,
                           (hipStream_t)stream, n, f);
        return check();
    }

    // dst[b][k][r] = src[b][r][k] for `batch` matrices of R x K elements of esz (2 or 4) bytes
    static int transpose(const void *src, void *dst, long long batch, long long R, long long K,
                         int esz, void *stream)
    {
        if (batch <= 0 || R <= 0 || K <= 0) return 0;
        const bool pairs = esz == 2 && R % 2 == 0 && K % 2 == 0 && (((uintptr_t)src | (uintptr_t)dst) & 3u) == 0;
        const long long t = pairs ? 64 : 32;
        const long long tiles_r = (R + t - 1) / t, tiles_k = (K + t - 1) / t;
        const long long nblk = batch * tiles_r * tiles_k;
        if (nblk > 0x7fffffffLL) return -2;
        if (pairs)
            hipLaunchKernelGGL(transpose_pairs_kernel, dim3((unsigned)nblk), dim3(256), 0, (hipStream_t)stream,
                               (const uint32_t *)src, (uint32_t *)dst, R, K, tiles_r, tiles_k);
        else if (esz == 2)
            hipLaunchKernelGGL(transpose_kernel<uint16_t>, dim3((unsigned)nblk), dim3(256), 0,
                               (hipStream_t)stream, (const uint16_t *)src, (uint16_t *)dst, R, K, tiles_r, tiles_k);
        else
            hipLaunchKernelGGL(transpose_kernel<uint32_t>, dim3((unsigned)nblk), dim3(256), 0,
                               (hipStream_t)stream, (const uint32_t *)src, (uint32_t *)dst, R, K, tiles_r, tiles_k);
        return check();
    }

    // Row normalisation, one direction: reduce launch then apply launch on rows * nsplit
    // workgroups.  Forward: a = x, out = y, stats written; backward: a = gy, b = y, stats read,
    // out = gx.  `vec`: n is a multiple of 16 bytes of elements and every pointer is 16-byte
    // aligned.
    template <typename T, bool BWD, bool VEC>
    static void rownorm_launch(const void *a, const void *b, const void *addend, float *partial, float *stats,
                               void *out, long long rows, const rownorm::Split &sp, float eps, void *stream)
    {
        using namespace rownorm;
        const dim3 grid((unsigned)(rows * sp.nsplit)), block(kThreads);
        hipLaunchKernelGGL((reduce_kernel<T, BWD, VEC>), grid, block, 0, (hipStream_t)stream, (const T *)a,
                           (const T *)b, (float2 *)partial, sp);
        if (BWD && addend)
            hipLaunchKernelGGL((apply_kernel<T, BWD, VEC, BWD>), grid, block, 0, (hipStream_t)stream, (const T *)a,
                               (const T *)b, (const T *)addend, (const float2 *)partial, (float2 *)stats, (T *)out,
                               sp, eps);
        else
            hipLaunchKernelGGL((apply_kernel<T, BWD, VEC, false>), grid, block, 0, (hipStream_t)stream,
                               (const T *)a, (const T *)b, (const T *)nullptr, (const float2 *)partial,
                               (float2 *)stats, (T *)out, sp, eps);
    }

    // Row normalisation, one direction: reduce launch then apply launch on rows * nsplit
    // workgroups.  Forward: a = x, out = y, stats written; backward: a = gy, b = y, stats read,
    // out = gx (+ addend, if given).  `vec`: n is a multiple of 16 bytes of elements and every
    // pointer is 16-byte aligned.
    template <typename T>
    static void rownorm_t(bool bwd, const void *a, const void *b, const void *addend, float *partial, float *stats,
                          void *out, long long rows, const rownorm::Split &sp, bool vec, float eps, void *stream)
    {
        if (bwd) {
            if (vec) rownorm_launch<T, true, true>(a, b, addend, partial, stats, out, rows, sp, eps, stream);
            else rownorm_launch<T, true, false>(a, b, addend, partial, stats, out, rows, sp, eps, stream);
        } else {
            if (vec) rownorm_launch<T, false, true>(a, b, addend, partial, stats, out, rows, sp, eps, stream);
            else rownorm_launch<T, false, false>(a, b, addend, partial, stats, out, rows, sp, eps, stream);
        }
    }

    static int rownorm(bool bwd, const void *a, const void *b, const void *addend, float *partial, float *stats,
                       void *out, long long rows, long long n, int nsplit, long long chunk, int esz, bool vec,
                       float eps, void *stream)
    {
        if (rows <= 0 || n <= 0) return 0;
        const rownorm::Split sp = {n, chunk, nsplit};
        if (esz == 2) rownorm_t<bf16_t>(bwd, a, b, addend, partial, stats, out, rows, sp, vec, eps, stream);
        else rownorm_t<float>(bwd, a, b, addend, partial, stats, out, rows, sp, vec, eps, stream);
        return check();
    }

    // normalisation over the channels of a channel-first (B, C, n) tensor; see ndc_chnorm.h
    static constexpr int kChnormWaves = rownorm::kThreads / 64;   // partial rows per workgroup
    static long long chnorm_blocks(long long n, int esz, bool vec)
    {
        const long long per = vec ? 16 / esz : 1;
        return (n / per + rownorm::kThreads - 1) / rownorm::kThreads;
    }
    template <typename T, bool VEC>
    static void chnorm_launch(bool bwd, const void *a, const void *x, const float *stats, const float *weight,
                              const float *bias, void *out, float *partial, long long B, int C, long long n,
                              float eps, void *stream)
    {
        const chnorm::Shape sh = {n, C, (int)chnorm_blocks(n, (int)sizeof(T), VEC)};
        const dim3 grid((unsigned)(B * sh.blocks)), block(rownorm::kThreads);
        if (bwd)
            hipLaunchKernelGGL((chnorm::backward_kernel<T, VEC>), grid, block, 0, (hipStream_t)stream, (const T *)a,
                               (const T *)x, stats, weight, (T *)out, partial, sh);
        else
            hipLaunchKernelGGL((chnorm::forward_kernel<T, VEC>), grid, block, 0, (hipStream_t)stream, (const T *)x,
                               weight, bias, (T *)out, const_cast<float *>(stats), sh, eps);
    }
    static int chnorm(bool bwd, const void *a, const void *x, const float *stats, const float *weight,
                      const float *bias, void *out, float *partial, long long B, int C, long long n, int esz,
                      bool vec, float eps, void *stream)
    {
        if (B <= 0 || C <= 0 || n <= 0) return 0;
        if (B * chnorm_blocks(n, esz, vec) > 0x7fffffffLL) return -2;
        if (esz == 2) {
            if (vec) chnorm_launch<bf16_t, true>(bwd, a, x, stats, weight, bias, out, partial, B, C, n, eps, stream);
            else chnorm_launch<bf16_t, false>(bwd, a, x, stats, weight, bias, out, partial, B, C, n, eps, stream);
        } else {
            if (vec) chnorm_launch<float, true>(bwd, a, x, stats, weight, bias, out, partial, B, C, n, eps, stream);
            else chnorm_launch<float, false>(bwd, a, x, stats, weight, bias, out, partial, B, C, n, eps, stream);
        }
        return check();
    }

    static int row_sums(const void *a, float *partial, long long rows, long long n, int nsplit, long long chunk,
                        int esz, bool vec, void *stream)
    {
        if (rows <= 0 || n <= 0) return 0;
        const rownorm::Split sp = {n, chunk, nsplit};
        const dim3 grid((unsigned)(rows * nsplit)), block(rownorm::kThreads);
        if (esz == 2) {
            if (vec) hipLaunchKernelGGL((rownorm::row_sums_kernel<bf16_t, true>), grid, block, 0, (hipStream_t)stream, (const bf16_t *)a, partial, sp);
            else hipLaunchKernelGGL((rownorm::row_sums_kernel<bf16_t, false>), grid, block, 0, (hipStream_t)stream, (const bf16_t *)a, partial, sp);
        } else {
            if (vec) hipLaunchKernelGGL((rownorm::row_sums_kernel<float, true>), grid, block, 0, (hipStream_t)stream, (const float *)a, partial, sp);
            else hipLaunchKernelGGL((rownorm::row_sums_kernel<float, false>), grid, block, 0, (hipStream_t)stream, (const float *)a, partial, sp);
        }
        return check();
    }

    // y = act(z + bias[channel]) + residual on rows * nsplit workgroups (bias, residual optional)
    template <typename T, int ACT, bool RES>
    static void bias_act_launch(const void *z, const float *bias, const void *res, void *y, int channels,
                                const rownorm::Split &sp, long long rows, bool vec, void *stream)
    {
        const dim3 grid((unsigned)(rows * sp.nsplit)), block(rownorm::kThreads);
        if (vec)
            hipLaunchKernelGGL((epilogue::forward_kernel<T, ACT, RES, true>), grid, block, 0, (hipStream_t)stream,
                               (const T *)z, bias, (const T *)res, (T *)y, channels, sp);
        else
            hipLaunchKernelGGL((epilogue::forward_kernel<T, ACT, RES, false>), grid, block, 0, (hipStream_t)stream,
                               (const T *)z, bias, (const T *)res, (T *)y, channels, sp);
    }

    template <typename T>
    static int bias_act_t(const void *z, const float *bias, const void *res, void *y, long long rows,
                          int channels, long long n, int nsplit, long long chunk, int act, bool vec, void *stream)
    {
        const rownorm::Split sp = {n, chunk, nsplit};
#define NDC_BIAS_ACT(ACT)                                                                        \
    (res ? bias_act_launch<T, ACT, true>(z, bias, res, y, channels, sp, rows, vec, stream)        \
         : bias_act_launch<T, ACT, false>(z, bias, res, y, channels, sp, rows, vec, stream))
        if (act == epilogue::kNone) NDC_BIAS_ACT(epilogue::kNone);
        else if (act == epilogue::kRelu) NDC_BIAS_ACT(epilogue::kRelu);
        else NDC_BIAS_ACT(epilogue::kGelu);
#undef NDC_BIAS_ACT
        return check();
    }

    static int bias_act(const void *z, const float *bias, const void *res, void *y, long long rows,
                        int channels, long long n, int nsplit, long long chunk, int act, int esz, bool vec,
                        void *stream)
    {
        if (rows <= 0 || n <= 0) return 0;
        return esz == 2 ? bias_act_t<bf16_t>(z, bias, res, y, rows, channels, n, nsplit, chunk, act, vec, stream)
                        : bias_act_t<float>(z, bias, res, y, rows, channels, n, nsplit, chunk, act, vec, stream);
    }

    template <typename T, int ACT>
    static void bias_act_bwd_launch(const void *gy, const void *z, const float *bias, void *gz, float *gpart,
                                    int channels, const rownorm::Split &sp, long long rows, bool vec, void *stream)
    {
        const dim3 grid((unsigned)(rows * sp.nsplit)), block(rownorm::kThreads);
        if (vec)
            hipLaunchKernelGGL((epilogue::backward_kernel<T, ACT, true>), grid, block, 0, (hipStream_t)stream,
                               (const T *)gy, (const T *)z, bias, (T *)gz, gpart, channels, sp);
        else
            hipLaunchKernelGGL((epilogue::backward_kernel<T, ACT, false>), grid, block, 0, (hipStream_t)stream,
                               (const T *)gy, (const T *)z, bias, (T *)gz, gpart, channels, sp);
    }

    // gz = gy * act'(z + bias), gpart[row * nsplit + part] = the part's sum of gz (act: relu, gelu)
    static int bias_act_backward(const void *gy, const void *z, const float *bias, void *gz, float *gpart,
                                 long long rows, int channels, long long n, int nsplit, long long chunk, int act,
                                 int esz, bool vec, void *stream)
    {
        if (rows <= 0 || n <= 0) return 0;
        const rownorm::Split sp = {n, chunk, nsplit};
        if (esz == 2) {
            if (act == epilogue::kRelu) bias_act_bwd_launch<bf16_t, epilogue::kRelu>(gy, z, bias, gz, gpart, channels, sp, rows, vec, stream);
            else bias_act_bwd_launch<bf16_t, epilogue::kGelu>(gy, z, bias, gz, gpart, channels, sp, rows, vec, stream);
        } else {
            if (act == epilogue::kRelu) bias_act_bwd_launch<float, epilogue::kRelu>(gy, z, bias, gz, gpart, channels, sp, rows, vec, stream);
            else bias_act_bwd_launch<float, epilogue::kGelu>(gy, z, bias, gz, gpart, channels, sp, rows, vec, stream);
        }
        return check();
    }

    // 2 x 2 (x 2) windows of a fine grid <-> 4 (8) planes of the coarse grid; see ndc_regroup.h
    static int regroup2(const void *src, void *dst, const float *bias, long long rows, int channels, int D,
                        int H, int W, int depth2, int esz, int to_channels, void *stream)
    {
        const regroup::Shape sh = {rows, D, H, W, depth2, channels};
        const long long nvec = rows * D * H * (W / (16 / esz));
        if (nvec <= 0) return 0;
        const long long blocks = (nvec + 255) / 256;
        if (blocks > 0x7fffffffLL) return -2;
        const dim3 grid((unsigned)blocks), block(256);
        if (esz == 2) {
            if (to_channels) hipLaunchKernelGGL((regroup::kernel<2, true>), grid, block, 0, (hipStream_t)stream, src, dst, bias, sh, nvec);
            else hipLaunchKernelGGL((regroup::kernel<2, false>), grid, block, 0, (hipStream_t)stream, src, dst, bias, sh, nvec);
        } else {
            if (to_channels) hipLaunchKernelGGL((regroup::kernel<4, true>), grid, block, 0, (hipStream_t)stream, src, dst, bias, sh, nvec);
            else hipLaunchKernelGGL((regroup::kernel<4, false>), grid, block, 0, (hipStream_t)stream, src, dst, bias, sh, nvec);
        }
        return check();
    }

    // weights (cout x cin, or the transpose stored as cin x cout) -> fragment order; see ndc_pwgemm.h
    static int pwgemm_pack(const void *w, int w_is_bf16, int transposed, void *wfrag, int cout, int cin, void *stream)
    {
        const long long n = (long long)(cout / 32) * (cin / 16) * 64;
        const dim3 grid((unsigned)((n + 255) / 256)), block(256);
        uint16_t *o = (uint16_t *)wfrag;
        if (w_is_bf16) {
            if (transposed) hipLaunchKernelGGL((pwgemm::pack_kernel<bf16_t, true>), grid, block, 0, (hipStream_t)stream, (const bf16_t *)w, o, cout, cin);
            else hipLaunchKernelGGL((pwgemm::pack_kernel<bf16_t, false>), grid, block, 0, (hipStream_t)stream, (const bf16_t *)w, o, cout, cin);
        } else {
            if (transposed) hipLaunchKernelGGL((pwgemm::pack_kernel<float, true>), grid, block, 0, (hipStream_t)stream, (const float *)w, o, cout, cin);
            else hipLaunchKernelGGL((pwgemm::pack_kernel<float, false>), grid, block, 0, (hipStream_t)stream, (const float *)w, o, cout, cin);
        }
        return check();
    }

    // persistent workgroups: as many as are resident at once (asked of the runtime once per
    // kernel and LDS size), so that every wavefront walks the same number of tiles
    template <int CIN, int ACT, bool RES, int THREADS>
    static int pwgemm_launch(const pwgemm::Params &p, size_t lds, void *stream)
    {
        void (*entry)(pwgemm::Params) = pwgemm::gemm_kernel<CIN, ACT, RES, THREADS>;
        static std::atomic<int> resident[3] = {{0}, {0}, {0}};   // by LDS size class
        const int cls = lds <= 40 * 1024 ? 0 : lds <= 80 * 1024 ? 1 : 2;
        int per_cu = resident[cls].load(std::memory_order_relaxed);
        if (per_cu == 0) {
            // (asked for the largest LDS size of the class, so that the answer holds for all of it)
            const size_t worst = cls == 0 ? 40 * 1024 : cls == 1 ? 80 * 1024 : 160 * 1024;
            if (worst > 64 * 1024 &&
                hipFuncSetAttribute((const void *)entry, hipFuncAttributeMaxDynamicSharedMemorySize, (int)worst) != hipSuccess)
                return -5;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)entry, THREADS, worst) != hipSuccess ||
                per_cu < 1)
                per_cu = 1;
            resident[cls].store(per_cu, std::memory_order_relaxed);
        }
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) == hipSuccess) {
            static std::atomic<int> cu_count{0};
            cus = cu_count.load(std::memory_order_relaxed);
            if (cus == 0) {
                if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
                cu_count.store(cus, std::memory_order_relaxed);
            }
        }
        long long blocks = (long long)cus * per_cu;
        const long long need = ((long long)p.tiles + THREADS / 64 - 1) / (THREADS / 64);
        if (blocks > need) blocks = need;
        // gradient modes: one row of sums per wavefront (the kernel zeroes the rows nobody owns)
        if (p.gpart && blocks * (THREADS / 64) > pwgemm::kMaxParts) blocks = pwgemm::kMaxParts / (THREADS / 64);
        hipLaunchKernelGGL(entry, dim3((unsigned)blocks), dim3(THREADS), lds, (hipStream_t)stream, p);
        return check();
    }

    template <int CIN, int THREADS>
    static int pwgemm_act(const pwgemm::Params &p, size_t lds, int act, void *stream)
    {
#define NDC_PWGEMM_RES(ACT)                                                                 \
    (p.res ? pwgemm_launch<CIN, ACT, true, THREADS>(p, lds, stream)                         \
           : pwgemm_launch<CIN, ACT, false, THREADS>(p, lds, stream))
        // gradient modes hold a row of sums per wavefront in LDS as well
        const size_t glds = lds + (size_t)(THREADS / 64) * p.cout * 4;
        if (act >= pwgemm::kReluGrad && glds > 160 * 1024) return -2;
        if (act == pwgemm::kGeluGrad) return pwgemm_launch<CIN, pwgemm::kGeluGrad, true, THREADS>(p, glds, stream);
        if (act == pwgemm::kReluGrad) return pwgemm_launch<CIN, pwgemm::kReluGrad, true, THREADS>(p, glds, stream);
        if (act == pwgemm::kMasked) return NDC_PWGEMM_RES(pwgemm::kMasked);
        if (act == epilogue::kRelu) return NDC_PWGEMM_RES(epilogue::kRelu);
        if (act == epilogue::kGelu) return NDC_PWGEMM_RES(epilogue::kGelu);
        return NDC_PWGEMM_RES(epilogue::kNone);
#undef NDC_PWGEMM_RES
    }

    // y = act(W x + bias) + residual on persistent workgroups; the caller has checked the shape
    // (cin in {64, 128, 256}, cout a multiple of 32, n a multiple of 64, packed weights <= 128 KB)
    template <int CT, bool RES, bool MASK>
    static int pwgemm_deep_launch(const pwgemm::Params &p, int cin, size_t lds, void *stream)
    {
        constexpr int THREADS = 512;
        void (*entry)(pwgemm::Params, int) = pwgemm::gemm_kernel_deep<CT, RES, MASK, THREADS>;
        static std::atomic<int> resident[2] = {{0}, {0}};
        const int cls = lds <= 72 * 1024 ? 0 : 1;
        int per_cu = resident[cls].load(std::memory_order_relaxed);
        if (per_cu == 0) {
            const size_t worst = cls == 0 ? 72 * 1024 : 160 * 1024;
            if (hipFuncSetAttribute((const void *)entry, hipFuncAttributeMaxDynamicSharedMemorySize, (int)worst) != hipSuccess)
                return -5;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)entry, THREADS, worst) != hipSuccess ||
                per_cu < 1)
                per_cu = 1;
            resident[cls].store(per_cu, std::memory_order_relaxed);
        }
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
            cus = 256;
        long long blocks = (long long)cus * per_cu;
        const long long need = ((long long)p.tiles + THREADS / 64 - 1) / (THREADS / 64);
        if (blocks > need) blocks = need;
        hipLaunchKernelGGL(entry, dim3((unsigned)blocks), dim3(THREADS), lds, (hipStream_t)stream, p, cin);
        return check();
    }

    template <int CT>
    static int pwgemm_deep(const pwgemm::Params &p, int cin, size_t lds, void *stream)
    {
        if (p.mask)
            return p.res ? pwgemm_deep_launch<CT, true, true>(p, cin, lds, stream)
                         : pwgemm_deep_launch<CT, false, true>(p, cin, lds, stream);
        return p.res ? pwgemm_deep_launch<CT, true, false>(p, cin, lds, stream)
                     : pwgemm_deep_launch<CT, false, false>(p, cin, lds, stream);
    }

    // act 3 / 4: y = (W x) * relu' / gelu'(res + bias), gpart (kMaxParts x cout, or null) receives
    // per-wavefront sums of y whose total over the rows is the bias gradient
    // act 5: y = (W x + bias + res) where mask > 0, else 0
    static int pwgemm(const void *x, const void *wfrag, const float *bias, const void *res, void *y, void *zkeep,
                      float *gpart, const void *mask, long long batch, int cin, int cout, long long n, int act,
                      void *stream)
    {
        pwgemm::Params p;
        p.gpart = gpart;
        p.mask = (const uint16_t *)mask;
        p.x = (const uint16_t *)x, p.wfrag = (const uint16_t *)wfrag, p.bias = bias;
        p.res = (const uint16_t *)res, p.y = (uint16_t *)y, p.zkeep = (uint16_t *)zkeep;
        p.n = n, p.tiles_per_sample = (int)(n / pwgemm::kTileVoxels), p.tiles = (int)(batch * (n / pwgemm::kTileVoxels)), p.cout = cout;
        if (p.tiles <= 0) return 0;
        const size_t wbytes = (size_t)cin * cout * 2;
        const size_t lds = wbytes + (size_t)cout * 4;   // packed weights, bias
        if (cin > 256) {   // many input channels, at most 128 output channels (checked by the caller)
            if ((act != epilogue::kNone && act != pwgemm::kMasked) || zkeep) return -2;   // product, bias, residual, mask
            switch (cout / 32) {
            case 1: return pwgemm_deep<1>(p, cin, lds, stream);
            case 2: return pwgemm_deep<2>(p, cin, lds, stream);
            case 3: return pwgemm_deep<3>(p, cin, lds, stream);
            default: return pwgemm_deep<4>(p, cin, lds, stream);
            }
        }
        // small weight tables: several workgroups per CU; large ones: one, of more wavefronts
        int threads = wbytes <= 32 * 1024 ? 256 : wbytes <= 64 * 1024 || cin == 256 ? 512 : 1024;
        if (act >= pwgemm::kReluGrad && lds + (size_t)(threads / 64) * cout * 4 > 160 * 1024) threads = 512;
#define NDC_PWGEMM(CIN)                                                                            \
    (threads == 256 ? pwgemm_act<CIN, 256>(p, lds, act, stream)                                     \
     : threads == 512 ? pwgemm_act<CIN, 512>(p, lds, act, stream)                                   \
                      : pwgemm_act<CIN, 1024>(p, lds, act, stream))
        if (cin == 64) return NDC_PWGEMM(64);
        if (cin == 128) return NDC_PWGEMM(128);
        return threads == 256 ? pwgemm_act<256, 256>(p, lds, act, stream) : pwgemm_act<256, 512>(p, lds, act, stream);
#undef NDC_PWGEMM
    }

    static constexpr int kSumSlices = 8;
    template <class P, class F> static int strided_sum(int nout, int nparts, void *stream, P put, F term)
    {
        if (nout <= 0) return 0;
        hipLaunchKernelGGL((strided_sum_kernel<P, F>), dim3((unsigned)((nout + 31) / 32)), dim3(256), 0,
                           (hipStream_t)stream, nout, nparts, put, term);
        return check();
    }

    template <class F> static int block_reduce(int nout, void *stream, float *out, F partial)
    {
        if (nout <= 0) return 0;
        hipLaunchKernelGGL(block_reduce_kernel<F>, dim3((unsigned)nout), dim3(256), 0,
                           (hipStream_t)stream, out, partial);
        return check();
    }
};

}  // namespace ndc

#include "ndc_api_impl.h"

// ============================================================================ no-allocation forward
//
// ndc_forward for callers that cannot hand over a workspace they allocated (code under graph
// capture that was set up without one, serving loops and harnesses that forbid hipMalloc):
// the forward's scratch -- the packed filter tables of the bfloat16 3x3x3 kernels -- lives in
// a file-scope device array instead.  Every GPU the library runs on holds its own copy of the
// array, at its own address, until the process ends.

#include <mutex>

namespace {

static __device__ __align__(256) unsigned char scratch[NDC_NOALLOC_SCRATCH_BYTES];

// In host code the name `scratch` is only a handle for hipGetSymbolAddress; the device
// address is looked up once per device (with that device current) and kept here.  Kernels,
// copies and memsets are always given this pointer, never the array's name.
const int kMaxDevices = 64;
void *scratch_dev_ptr[kMaxDevices] = {nullptr};
std::mutex scratch_mutex;

int scratch_address(void **out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return NDC_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_dev_ptr[dev]) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr)
            return NDC_ERR_LAUNCH;
        scratch_dev_ptr[dev] = ptr;
    }
    *out = scratch_dev_ptr[dev];
    return NDC_OK;
}

}  // namespace

extern "C" int ndc_noalloc_init(void)
{
    void *ptr = nullptr;
    return scratch_address(&ptr);
}

extern "C" int ndc_forward_noalloc(const ndc_geom *g, const void *x, const void *z, const float *h,
                                   const float *bias, void *out, void *t1, void *s_over_den,
                                   void *ratio, void *stream)
{
    ndc::KGeom q;
    const int st = ndc::make_kgeom(g, q);
    if (st) return st;
    const size_t need = ndc_forward_workspace_bytes(g);
    if (need > (size_t)NDC_NOALLOC_SCRATCH_BYTES) return NDC_ERR_SCRATCH_LIMIT;
    void *ptr = nullptr;
    if (need) {
        const int sa = scratch_address(&ptr);
        if (sa) return sa;
    }
    // the tables are rewritten in full by every call (nothing has to start at zero); the
    // launches that fill and read them are ordered on `stream`
    return ndc_forward(g, x, z, h, bias, out, t1, s_over_den, ratio, ptr,
                       need ? (size_t)NDC_NOALLOC_SCRATCH_BYTES : 0, stream);
}
