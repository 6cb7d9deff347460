// Sequential host build of the NDC C ABI.  Same kernel bodies and host logic as the HIP
// build, executed thread by thread on the CPU, so that the CPU test-suite can check
// indexing, bounds and barrier placement before anything runs on a GPU.  It is a checker
// for the kernels' source, not a fallback: the Python package never loads it.
#include <vector>

#include "ndc_common.h"

#define NDC_LAMBDA

namespace ndc {

struct Backend {
    static constexpr bool is_device = false;

    template <class F> static int elementwise(long long n, void *, F f)
    {
        for (long long idx = 0; idx < n; ++idx) f(idx);
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
