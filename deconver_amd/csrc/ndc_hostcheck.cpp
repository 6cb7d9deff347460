// Sequential host build of the NDC C ABI.  Same kernel bodies and host logic as the HIP
// build, executed thread by thread on the CPU, so that the CPU test-suite can check
// indexing, bounds and barrier placement before anything runs on a GPU.  It is a checker
// for the kernels' source, not a fallback: the Python package never loads it.
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
