// HIP (gfx950) build of the NDC C ABI: launch primitives + the shared host logic.
#include <hip/hip_runtime.h>

#include "ndc_common.h"

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

struct Backend {
    static constexpr bool is_device = true;

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
