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
#else
#define NDC_HD inline
#define NDC_D inline
#define NDC_DEVICE_BUILD 0
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
    uint32_t u;
#if NDC_DEVICE_BUILD && defined(__HIP_DEVICE_COMPILE__)
    u = __float_as_uint(f);
#else
    memcpy(&u, &f, 4);
#endif
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
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
    float eps;
    long long SP;  // D*H*W

    NDC_HD int C() const { return G * m; }
    NDC_HD int CS() const { return G * sc; }
};

}  // namespace ndc
