// Execution contexts of the block-cooperative (LDS-tiled) kernels.
//
// A kernel is written once as `Kernel::run(exec, params, block_id)`: a uniform sequence of
// per-thread phases (`exec.each(f)`) separated by barriers (`exec.sync()`), with all LDS
// traffic going through `exec.ld / exec.st`.  Two contexts implement that interface:
//
//   DeviceExec  one HIP thread: `each` runs the phase for this thread, `sync` is
//               __syncthreads(), ld/st are plain LDS accesses.
//   HostExec    a whole block on the CPU: `each` runs the phase for every thread in turn,
//               `sync` opens a new epoch, and ld/st are bounds-checked and race-checked:
//               two different threads touching one LDS word within an epoch, at least one
//               of them writing, is reported (it would need a barrier on the GPU), as is a
//               read of a word nobody has written.
#pragma once

#include "ndc_common.h"

#if !NDC_DEVICE_BUILD
#include <cstdio>
#include <cstring>
#include <vector>
#endif

namespace ndc {

#if NDC_DEVICE_BUILD

template <class State> struct DeviceExec {
    State st;
    float *lds;
    int tid;
    int nthreads;
    template <class F> NDC_D void each(F f) { f(st, tid); }
    NDC_D void sync() { __syncthreads(); }
    NDC_D float ld(int i) const { return lds[i]; }
    NDC_D void st_(int i, float v) { lds[i] = v; }
    // two consecutive words from an EVEN word index: one 8-byte read
    NDC_D void ld2(int i, float (&v)[2]) const
    {
        typedef __attribute__((ext_vector_type(2))) float f2_t;
        const f2_t a = *reinterpret_cast<const f2_t *>(lds + i);
        v[0] = a.x;
        v[1] = a.y;
    }
    // four consecutive words from an EVEN word index, as two 8-byte reads (one ds_read2_b64
    // where the compiler pairs them) instead of four 4-byte ones
    NDC_D void ld4(int i, uint32_t (&v)[4]) const
    {
        typedef __attribute__((ext_vector_type(2))) uint32_t u2_t;
        const u2_t a = *reinterpret_cast<const u2_t *>(lds + i);
        const u2_t b = *reinterpret_cast<const u2_t *>(lds + i + 2);
        v[0] = a.x;
        v[1] = a.y;
        v[2] = b.x;
        v[3] = b.y;
    }
    // four consecutive words from a word index that is a multiple of 4: one 16-byte read
    NDC_D void ld4a(int i, uint32_t (&v)[4]) const
    {
        typedef __attribute__((ext_vector_type(4))) uint32_t u4_t;
        const u4_t a = *reinterpret_cast<const u4_t *>(lds + i);
        v[0] = a.x;
        v[1] = a.y;
        v[2] = a.z;
        v[3] = a.w;
    }
    // two words to an EVEN word index: one 8-byte write
    NDC_D void st2(int i, uint32_t a, uint32_t b)
    {
        typedef __attribute__((ext_vector_type(2))) uint32_t u2_t;
        const u2_t v = {a, b};
        *reinterpret_cast<u2_t *>(lds + i) = v;
    }
    NDC_D void stw(int i, uint32_t a) { lds[i] = __uint_as_float(a); }
    // two consecutive words from any word index (one ds_read2_b32)
    NDC_D void ld2w(int i, uint32_t (&v)[2]) const
    {
        v[0] = __float_as_uint(lds[i]);
        v[1] = __float_as_uint(lds[i + 1]);
    }
    // The instruction scheduler may not move anything across this point: used to keep the LDS
    // reads of the next row ahead of the arithmetic on the current one.
    NDC_D void fence() const { __builtin_amdgcn_sched_barrier(0); }
    // The word `get(state)` of the lane to the left (lane - 1 of the wavefront); lane 0 gets 0.
    // For values a kernel computes (nothing in memory to fetch them from again).
    template <class G> NDC_D uint32_t left_lane(G get)
    {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)get(st), 0x138 /* wave_shr:1 */, 0xf, 0xf, true);
    }
    // every global load this thread has issued has returned (s_waitcnt vmcnt(0))
    NDC_D void wait_loads() const { __builtin_amdgcn_s_waitcnt(0x0F70); }

    // Sum N per-thread values over the workgroup: butterfly inside each wavefront, one LDS
    // row per wavefront, then thread i < N adds the rows in a fixed order and hands the sum
    // to `put`.  Reuses LDS from offset 0 (callers are done with their tiles by then).
    template <int N, class Get, class Put> NDC_D void block_reduce(Get get, Put put)
    {
        __syncthreads();
        const int lane = tid & 63, wave = tid >> 6, nw = nthreads >> 6;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            float v = get(st, i);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            if (lane == 0) lds[wave * N + i] = v;
        }
        __syncthreads();
        for (int i = tid; i < N; i += nthreads) {
            float s = 0.f;
            for (int w = 0; w < nw; ++w) s += lds[w * N + i];
            put(i, s);
        }
    }
};

#else

struct HostFaults {
    long long races = 0, oob = 0, uninit = 0;
    char first[256] = {0};
    void note(const char *what, int idx, int tid, int other)
    {
        if (!first[0]) snprintf(first, sizeof first, "%s at lds[%d] tid %d vs %d", what, idx, tid, other);
    }
};

inline HostFaults &host_faults()
{
    static HostFaults f;
    return f;
}

template <class State> struct HostExec {
    std::vector<State> states;
    std::vector<float> mem;
    std::vector<int> w_epoch, w_tid, r_epoch, r_tid;
    int nthreads;
    int cur = 0;
    int epoch = 0;

    HostExec(int nthreads_, int lds_floats)
        : states(nthreads_), mem(lds_floats, 0.f), w_epoch(lds_floats, -1), w_tid(lds_floats, -1),
          r_epoch(lds_floats, -1), r_tid(lds_floats, -1), nthreads(nthreads_)
    {
    }

    template <class F> void each(F f)
    {
        for (cur = 0; cur < nthreads; ++cur) f(states[cur], cur);
    }
    void sync() { ++epoch; }
    void fence() const {}
    void wait_loads() const {}
    // threads of a phase run in order, so the left neighbour has already computed its word
    // (both must have taken the same path through the phase up to here)
    template <class G> uint32_t left_lane(G get) { return cur & 63 ? get(states[cur - 1]) : 0u; }

    float ld(int i)
    {
        HostFaults &hf = host_faults();
        if (i < 0 || i >= (int)mem.size()) {
            ++hf.oob;
            hf.note("out-of-bounds read", i, cur, -1);
            return 0.f;
        }
        if (w_epoch[i] < 0) {
            ++hf.uninit;
            hf.note("uninitialised read", i, cur, -1);
        } else if (w_epoch[i] == epoch && w_tid[i] != cur) {
            ++hf.races;
            hf.note("read-after-write race", i, cur, w_tid[i]);
        }
        if (r_epoch[i] != epoch) {
            r_epoch[i] = epoch;
            r_tid[i] = cur;
        } else if (r_tid[i] != cur) {
            r_tid[i] = -2;
        }
        return mem[i];
    }
    void ld2(int i, float (&v)[2])
    {
        if (i & 1) {
            HostFaults &hf = host_faults();
            ++hf.oob;
            hf.note("misaligned two-word read", i, cur, -1);
        }
        v[0] = ld(i);
        v[1] = ld(i + 1);
    }
    void ld4(int i, uint32_t (&v)[4])
    {
        if (i & 1) {
            HostFaults &hf = host_faults();
            ++hf.oob;
            hf.note("misaligned four-word read", i, cur, -1);
        }
        for (int u = 0; u < 4; ++u) {
            const float f = ld(i + u);
            memcpy(&v[u], &f, 4);
        }
    }
    void ld4a(int i, uint32_t (&v)[4])
    {
        if (i & 3) {
            HostFaults &hf = host_faults();
            ++hf.oob;
            hf.note("misaligned 16-byte read", i, cur, -1);
        }
        for (int u = 0; u < 4; ++u) {
            const float f = ld(i + u);
            memcpy(&v[u], &f, 4);
        }
    }
    void ld2w(int i, uint32_t (&v)[2])
    {
        for (int u = 0; u < 2; ++u) {
            const float f = ld(i + u);
            memcpy(&v[u], &f, 4);
        }
    }
    void stw(int i, uint32_t a)
    {
        float f;
        memcpy(&f, &a, 4);
        st_(i, f);
    }
    void st2(int i, uint32_t a, uint32_t b)
    {
        if (i & 1) {
            HostFaults &hf = host_faults();
            ++hf.oob;
            hf.note("misaligned 8-byte write", i, cur, -1);
        }
        stw(i, a);
        stw(i + 1, b);
    }
    void st_(int i, float v)
    {
        HostFaults &hf = host_faults();
        if (i < 0 || i >= (int)mem.size()) {
            ++hf.oob;
            hf.note("out-of-bounds write", i, cur, -1);
            return;
        }
        if (w_epoch[i] == epoch && w_tid[i] != cur) {
            ++hf.races;
            hf.note("write-after-write race", i, cur, w_tid[i]);
        }
        if (r_epoch[i] == epoch && r_tid[i] != cur) {
            ++hf.races;
            hf.note("write-after-read race", i, cur, r_tid[i]);
        }
        w_epoch[i] = epoch;
        w_tid[i] = cur;
        mem[i] = v;
    }

    template <int N, class Get, class Put> void block_reduce(Get get, Put put)
    {
        sync();
        for (int i = 0; i < N; ++i) {
            float s = 0.f;
            for (int t = 0; t < nthreads; ++t) s += get(states[t], i);
            put(i, s);
        }
    }
};

#endif

// A slice of a tensor in global memory, addressed as (slice base, wave-uniform byte offset,
// per-lane byte offset), for 32-bit accesses.
//   Device: a raw buffer resource of `bytes` bytes.  The memory unit adds the three parts
//     (buffer_load_dword v, v_lane_off, s[resource], s_uniform_off offen), so no vector
//     instruction is spent on 64-bit address arithmetic, and an access past `bytes` is
//     dropped (loads return 0) instead of faulting.  A null base gives an empty slice.
//   Host build: base pointer + size; an access outside the slice is reported as a fault.
// A per-lane offset that lies outside every slice (slices addressed this way are kept below
// 2^31 bytes): a lane that has nothing to read or write at some row uses it instead of a
// branch or a select, and gets 0 from a load and no effect from a store.
static const unsigned kNoAccess = 0x80000000u;

struct BufRef {
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    __amdgpu_buffer_rsrc_t r;
#else
    char *base;
    size_t bytes;
#endif
};

NDC_HD BufRef make_buf(const void *p, size_t bytes)
{
    BufRef b;
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    // the slice base is the same in every lane: say so, or each access is wrapped in a loop
    // over the distinct resources of the wavefront
    const unsigned long long a = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    void *up = (void *)(((unsigned long long)hi << 32) | lo);
    const int n = __builtin_amdgcn_readfirstlane(p ? (int)(unsigned)bytes : 0);
    // word 3 of the resource: 32-bit data format, raw (unstrided, unswizzled) addressing
    b.r = __builtin_amdgcn_make_buffer_rsrc(up, 0, n, 0x00020000);
#else
    b.base = (char *)const_cast<void *>(p);
    b.bytes = p ? bytes : 0;
#endif
    return b;
}

// STREAM: the word is read once (non-temporal hint, as for buf_st).
template <bool STREAM = false>
NDC_HD uint32_t buf_ld(const BufRef &b, unsigned lane_off, unsigned uniform_off)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_raw_buffer_load_b32(b.r, (int)lane_off, (int)uniform_off, STREAM ? 2 : 0);
#elif NDC_DEVICE_BUILD
    (void)b; (void)lane_off; (void)uniform_off;
    return 0u;
#else
    if (lane_off >= kNoAccess || b.base == nullptr) return 0u;   // by design: nothing there
    const size_t o = (size_t)lane_off + uniform_off;
    if (o + 4 > b.bytes) {
        HostFaults &hf = host_faults();
        ++hf.oob;
        hf.note("out-of-bounds global read", (int)o, -1, -1);
        return 0u;
    }
    uint32_t w;
    memcpy(&w, b.base + o, 4);
    return w;
#endif
}

// STREAM: the word is not read again soon (a result tensor): stored with the non-temporal
// hint, so that it does not push re-used lines out of the L2.
template <bool STREAM = false>
NDC_HD void buf_st(const BufRef &b, unsigned lane_off, unsigned uniform_off, uint32_t w)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_buffer_store_b32(w, b.r, (int)lane_off, (int)uniform_off, STREAM ? 2 : 0);
#elif NDC_DEVICE_BUILD
    (void)b; (void)lane_off; (void)uniform_off; (void)w;
#else
    if (lane_off >= kNoAccess || b.base == nullptr) return;   // by design: goes nowhere
    const size_t o = (size_t)lane_off + uniform_off;
    if (o + 4 > b.bytes) {
        HostFaults &hf = host_faults();
        ++hf.oob;
        hf.note("out-of-bounds global write", (int)o, -1, -1);
        return;
    }
    memcpy(b.base + o, &w, 4);
#endif
}

}  // namespace ndc
