// Shared definitions of the NDC kernels.  Every kernel body in this directory is written
// once and compiled twice: by hipcc for gfx950 (the product) and by g++ as a sequential
// host build that the CPU test-suite uses to check indexing and barrier placement.
#pragma once

#include <stddef.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define NDC_HD __host__ __device__ __forceinline__
#define NDC_D __device__ __forceinline__
#define NDC_DEVICE_BUILD 1
// kernel-body lambdas are inlined before any per-function optimisation, so that the
// per-thread state they take by reference is promoted to registers as one object
#define NDC_LAMBDA __attribute__((always_inline))
#else
#define NDC_HD inline
#define NDC_D inline
#define NDC_DEVICE_BUILD 0
#define NDC_LAMBDA
#endif

namespace ndc {

typedef uint16_t bf16_t;  // raw bfloat16 bits

NDC_HD float bf16_to_float(bf16_t v)
{
    uint32_t u = (uint32_t)v << 16;
    float f;
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    f = __uint_as_float(u);
#else
    memcpy(&f, &u, 4);
#endif
    return f;
}

// round-to-nearest-even, NaN kept quiet
NDC_HD bf16_t float_to_bf16(float f)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(bf16_t, (__bf16)f);   // v_cvt_pk_bf16_f32
#else
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
#endif
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static NDC_HD float load(const float *p) { return *p; }
    static NDC_HD void store(float *p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    static NDC_HD float load(const bf16_t *p) { return bf16_to_float(*p); }
    static NDC_HD void store(bf16_t *p, float v) { *p = float_to_bf16(v); }
};

// two floats -> packed bf16 pair (lo in bits 0-15): one v_cvt_pk_bf16_f32 on gfx950
NDC_HD uint32_t pack_bf16x2(float lo, float hi)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((ext_vector_type(2))) float f2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf2_t;
    const f2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2_t));
#else
    return (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
#endif
}

NDC_HD float bits_to_float(uint32_t u)
{
    float f;
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    f = __uint_as_float(u);
#else
    memcpy(&f, &u, 4);
#endif
    return f;
}

NDC_HD uint32_t float_to_bits(float f)
{
    uint32_t u;
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    u = __float_as_uint(f);
#else
    memcpy(&u, &f, 4);
#endif
    return u;
}

// acc + a.lo*b.lo + a.hi*b.hi on packed bf16 pairs, float32 accumulate: one
// v_dot2c_f32_bf16 (issues at the rate of an fp32 FMA, i.e. two MACs per lane-instruction)
NDC_HD float dot2_bf16(uint32_t a, uint32_t b, float acc)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((ext_vector_type(2))) __bf16 bf2_t;
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2_t, a), __builtin_bit_cast(bf2_t, b),
                                           acc, false);
#else
    const float alo = bits_to_float(a << 16), ahi = bits_to_float(a & 0xffff0000u);
    const float blo = bits_to_float(b << 16), bhi = bits_to_float(b & 0xffff0000u);
    return acc + alo * blo + ahi * bhi;
#endif
}

// init + a.lo*b.lo + a.hi*b.hi with `b` a wave-uniform word: the three-operand
// v_dot2_f32_bf16, for the FIRST term of an accumulation.  The two-operand form the compiler
// selects for dot2_bf16 accumulates in place, so starting a sum from a value held elsewhere
// costs it a register copy per accumulator first; this form reads `init` where it lies.
NDC_HD float dot2_bf16_from(uint32_t a, uint32_t b_uniform, float init)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    float r;
    asm("v_dot2_f32_bf16 %0, %1, %2, %3" : "=v"(r) : "s"(b_uniform), "v"(a), "v"(init));
    return r;
#else
    return dot2_bf16(a, b_uniform, init);
#endif
}

// ---------------------------------------------------------------- 4x4x4 matrix instruction
//
// v_mfma_f32_4x4x4_16b_bf16 works on 16 independent blocks of 4 lanes.  In block b,
//   D[m][n] += sum_{k<4} A[m][k] * B[k][n],
// lane (b, m) = 4b + m holding row m of A as four bf16 (k = 0, 1 in its first word, k = 2, 3
// in its second), lane (b, n) holding column n of B the same way and receiving column n of D
// (m = 0..3 in four consecutive registers).  Products are exact, sums are float32.  One
// instruction does 16 * 64 multiply-accumulates and issues in about 10 clocks, against 128 in
// 4.5 for v_dot2c_f32_bf16.
//
// The kernels use it with lane <-> voxel column for B and D, and with rows of A that are a
// function of (block, m) which ANY lane can evaluate (filter taps from a table, staged words
// from LDS).  That is what lets the sequential host build check the same source: there a
// thread computes its own column of D from its own B and all four rows of A of its block.
typedef float f4_t __attribute__((vector_size(16)));

#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
struct MfmaRows {
    uint32_t w[2];   // this lane's row of A
};
// row(m, w): the two words of row m of A in the calling lane's block
template <class F> NDC_D void mfma_rows(MfmaRows &a, int lane, F row) { row(lane & 3, a.w); }
// row4(m, w): four words of row m, the rows of two matrices side by side
template <class F> NDC_D void mfma_rows2(MfmaRows &a0, MfmaRows &a1, int lane, F row4)
{
    uint32_t w[4];
    row4(lane & 3, w);
    a0.w[0] = w[0];
    a0.w[1] = w[1];
    a1.w[0] = w[2];
    a1.w[1] = w[3];
}
NDC_D void mfma_bf16_4x4x4(f4_t &acc, const MfmaRows &a, uint32_t b0, uint32_t b1)
{
    typedef short s4_t __attribute__((ext_vector_type(4)));
    typedef uint32_t u2_t __attribute__((ext_vector_type(2)));
    const u2_t av = {a.w[0], a.w[1]}, bv = {b0, b1};
    acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s4_t, av),
                                                 __builtin_bit_cast(s4_t, bv), acc, 0, 0, 0);
}
#else
struct MfmaRows {
    uint32_t w[4][2];   // all four rows of A of this lane's block
};
template <class F> NDC_D void mfma_rows(MfmaRows &a, int lane, F row)
{
    (void)lane;
    for (int m = 0; m < 4; ++m) row(m, a.w[m]);
}
template <class F> NDC_D void mfma_rows2(MfmaRows &a0, MfmaRows &a1, int lane, F row4)
{
    (void)lane;
    for (int m = 0; m < 4; ++m) {
        uint32_t w[4];
        row4(m, w);
        a0.w[m][0] = w[0];
        a0.w[m][1] = w[1];
        a1.w[m][0] = w[2];
        a1.w[m][1] = w[3];
    }
}
NDC_D void mfma_bf16_4x4x4(f4_t &acc, const MfmaRows &a, uint32_t b0, uint32_t b1)
{
    for (int m = 0; m < 4; ++m) {
        float s = acc[m];
        s += bits_to_float(a.w[m][0] << 16) * bits_to_float(b0 << 16);
        s += bits_to_float(a.w[m][0] & 0xffff0000u) * bits_to_float(b0 & 0xffff0000u);
        s += bits_to_float(a.w[m][1] << 16) * bits_to_float(b1 << 16);
        s += bits_to_float(a.w[m][1] & 0xffff0000u) * bits_to_float(b1 & 0xffff0000u);
        acc[m] = s;
    }
}
#endif

// The word the lane to the left (lane - 1 of the wavefront) holds in `own`; lane 0 gets 0.
// One v_mov_b32 with a wavefront shift.  `again` recomputes that word from memory: used by
// the sequential host build only, where lanes do not run side by side.
template <class F> NDC_D uint32_t from_left_lane(uint32_t own, F again)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    (void)again;
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own, 0x138 /* wave_shr:1 */, 0xf, 0xf, true);
#else
    (void)own;
    return again();
#endif
}

// N consecutive elements <-> N floats with one memory access (N = 1 or 2; the address must
// be aligned to N elements)
template <typename T, int N> struct VecIO;
template <typename T> struct VecIO<T, 1> {
    static NDC_HD void load(const T *p, float (&v)[1]) { v[0] = Elem<T>::load(p); }
    static NDC_HD void store(T *p, const float (&v)[1]) { Elem<T>::store(p, v[0]); }
};
template <> struct VecIO<float, 2> {
    struct alignas(8) Pair {
        float a, b;
    };
    static NDC_HD void load(const float *p, float (&v)[2])
    {
        const Pair q = *reinterpret_cast<const Pair *>(p);
        v[0] = q.a;
        v[1] = q.b;
    }
    static NDC_HD void store(float *p, const float (&v)[2])
    {
        Pair q;
        q.a = v[0];
        q.b = v[1];
        *reinterpret_cast<Pair *>(p) = q;
    }
};
template <> struct VecIO<bf16_t, 2> {
    static NDC_HD void load(const bf16_t *p, float (&v)[2])
    {
        const uint32_t w = *reinterpret_cast<const uint32_t *>(p);
        v[0] = bits_to_float(w << 16);
        v[1] = bits_to_float(w & 0xffff0000u);
    }
    static NDC_HD void store(bf16_t *p, const float (&v)[2])
    {
        *reinterpret_cast<uint32_t *>(p) = pack_bf16x2(v[0], v[1]);
    }
};

// max(v, 0): one v_max_f32 (a compare + select pair otherwise)
NDC_HD float relu_f(float v)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_fmaxf(v, 0.f);
#else
    return v > 0.f ? v : 0.f;
#endif
}

// max(v, lo) that hands a NaN in v on (as torch.relu does; fmaxf would return lo): one
// v_maximum3_f32.  With lo = kPassThrough it is the identity for every v, -inf included.
NDC_HD float floor_f(float v, float lo)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_elementwise_maximum(v, lo);
#else
    return v != v ? v : (v > lo ? v : lo);
#endif
}

NDC_HD float pass_through_floor()
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return -__builtin_huge_valf();
#else
    return -__builtin_huge_valf();
#endif
}

NDC_HD float fast_rcp(float v)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_rcpf(v);
#else
    return 1.0f / v;
#endif
}

// Read-only, wave-uniform data (filter taps, bias): on the device the pointer is re-typed
// into the constant address space, which lets the compiler fetch through the scalar unit
// (s_load into SGPRs) instead of issuing a vector load per lane.  The data must not be
// written by the kernel that reads it this way.
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
typedef const float __attribute__((address_space(4))) *UniformF;
NDC_D UniformF as_uniform(const float *p) { return (UniformF)(unsigned long long)p; }
#else
typedef const float *UniformF;
NDC_HD UniformF as_uniform(const float *p) { return p; }
#endif

// Tell the compiler that a value is the same in every lane (so that addresses derived from
// it stay on the scalar unit).
NDC_HD int uniform_int(int v)
{
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_readfirstlane(v);
#else
    return v;
#endif
}

template <int N> struct IntTag {
    static constexpr int value = N;
};

// Geometry as the kernels see it (derived once on the host from ndc_geom).
struct KGeom {
    int B, G, m, sc;
    int D, H, W;
    int kD, kH, kW;
    int pD, pH, pW;
    int KT;        // kD*kH*kW
    int relu;      // rectify z (+bias) on load
    int matrix;    // bf16 3x3x3 calls run the matrix-instruction kernel family where it covers them
    float eps;
    long long SP;  // D*H*W

    NDC_HD int C() const { return G * m; }
    NDC_HD int CS() const { return G * sc; }
};

}  // namespace ndc
