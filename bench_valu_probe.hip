// Instruction-issue probe for one MI355X: how many clocks a SIMD spends per wavefront
// instruction for the multiply-accumulate forms the NDC kernels can be built from, and what
// scalar, LDS and cross-lane instructions cost beside a stream of them.  This is the vector
// ceiling the update kernels are measured against (they are not HBM-bound): the kernels'
// v_dot2c_f32_bf16 count times the probed clocks per instruction is the least time the
// multiply-accumulates alone can take.
//
// Prints one JSON object.  Every kernel runs a fixed instruction stream on registers only
// (plus one LDS word per thread in the LDS row), 256 threads per workgroup.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

namespace {

enum Op {
    DOT2_SGPR, DOT2_VGPR, FMAC_SGPR, FMAC_VGPR, MUL_VGPR, ADD_VGPR, MAX_VGPR, CVT_PK_BF16, AND_VGPR,
    LSHL16, PERM, MOV_SGPR, READLANE,
    MIX_NONE, MIX_SMOV, MIX_LDS, MIX_WAITCNT, MIX_READLANE
};

// 8 x 16 instructions of the probed form per loop iteration; for the MIX_* forms the
// stream is v_dot2c with one other instruction after every fourth.
template <int OP> __global__ void __launch_bounds__(256) probe(float *out, const unsigned *w, int iters)
{
    __shared__ float lds[256];
    lds[threadIdx.x] = (float)threadIdx.x;
    __syncthreads();
    float acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = threadIdx.x * 0.001f + i;
    float x = threadIdx.x * 1.5f + 1.f;
    unsigned s[8];
    float v[8];
    for (int i = 0; i < 8; ++i) {
        s[i] = __builtin_amdgcn_readfirstlane(w[i]);
        v[i] = __uint_as_float(w[i] + threadIdx.x);
    }
    unsigned sink = 0, addr = threadIdx.x * 4;
    float lv = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
#define NDC_PROBE(id, text) \
    if (OP == id) asm volatile(text : "+v"(acc[i]) : "s"(s[(r + i) & 7]), "v"(v[(r + i) & 7]), "v"(x))
                NDC_PROBE(DOT2_SGPR, "v_dot2c_f32_bf16 %0, %1, %3");
                NDC_PROBE(DOT2_VGPR, "v_dot2c_f32_bf16 %0, %2, %3");
                NDC_PROBE(FMAC_SGPR, "v_fmac_f32 %0, %1, %3");
                NDC_PROBE(FMAC_VGPR, "v_fmac_f32 %0, %2, %3");
                NDC_PROBE(MUL_VGPR, "v_mul_f32 %0, %2, %3");
                NDC_PROBE(ADD_VGPR, "v_add_f32 %0, %2, %0");
                NDC_PROBE(MAX_VGPR, "v_max_f32 %0, %2, %0");
                NDC_PROBE(CVT_PK_BF16, "v_cvt_pk_bf16_f32 %0, %2, %0");
                NDC_PROBE(AND_VGPR, "v_and_b32 %0, %2, %0");
                NDC_PROBE(LSHL16, "v_lshlrev_b32 %0, 16, %0");
                NDC_PROBE(PERM, "v_perm_b32 %0, %2, %3, %0");
                NDC_PROBE(MOV_SGPR, "v_mov_b32 %0, %1");
#undef NDC_PROBE
                if (OP == READLANE) asm volatile("v_readlane_b32 %0, %1, 3" : "=s"(sink) : "v"(acc[i]));
                if (OP >= MIX_NONE) {
                    asm volatile("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(acc[i]) : "s"(s[(r + i) & 7]), "v"(x));
                    if ((i & 3) == 3) {
                        if (OP == MIX_SMOV) asm volatile("s_mov_b32 %0, %1" : "=s"(sink) : "s"(s[i & 7]));
                        if (OP == MIX_LDS) asm volatile("ds_read_b32 %0, %1" : "=v"(lv) : "v"(addr));
                        if (OP == MIX_WAITCNT) asm volatile("s_waitcnt lgkmcnt(0)");
                        if (OP == MIX_READLANE) asm volatile("v_readlane_b32 %0, %1, 0" : "=s"(sink) : "v"(x));
                    }
                }
            }
            if (OP == MIX_LDS) asm volatile("s_waitcnt lgkmcnt(0)");
        }
    }
    float t = lv + (float)sink;
    for (int i = 0; i < 16; ++i) t += acc[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = t;
}

// The 4x4x4 bf16 matrix instruction (1024 multiply-accumulates per wavefront instruction) alone
// and beside float32 FMAs, and LDS reads / writes of 4, 8 and 16 bytes per lane (dense,
// conflict-free addresses) with all four SIMDs of a CU issuing them: 4 x 8 instructions of the
// probed form per loop iteration.
enum Op2 { MFMA, MFMA_FMA1, MFMA_FMA2, LDS_R32, LDS_R64, LDS_R128, LDS_W32, LDS_W64, LDS_W128 };
typedef short probe_s4 __attribute__((ext_vector_type(4)));
typedef float probe_f4 __attribute__((ext_vector_type(4)));
typedef unsigned probe_u4 __attribute__((ext_vector_type(4)));
typedef unsigned probe_u2 __attribute__((ext_vector_type(2)));

template <int OP> __global__ void __launch_bounds__(256) probe2(float *out, const unsigned *w, int iters)
{
    __shared__ unsigned lds[256 * 4];
    for (int i = 0; i < 4; ++i) lds[threadIdx.x * 4 + i] = threadIdx.x;
    __syncthreads();
    probe_f4 acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = probe_f4{0.f, 1.f, 2.f, (float)i};
    probe_s4 a[4], b[4];
    for (int i = 0; i < 4; ++i) {
        a[i] = probe_s4{(short)w[i], (short)(w[i] + 1), (short)threadIdx.x, 3};
        b[i] = probe_s4{(short)w[i + 4], (short)(w[i] + 1), (short)threadIdx.x, 3};
    }
    float va[8];
    for (int i = 0; i < 8; ++i) va[i] = threadIdx.x + i;
    const float x = threadIdx.x * 1.5f + 1.f;
    const unsigned t = threadIdx.x;
    probe_u4 v4 = {t, t, t, t};
    probe_u2 v2 = {t, t};
    unsigned v1 = t;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if (OP <= MFMA_FMA2)
                    asm volatile("v_mfma_f32_4x4x4_16b_bf16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[(r + i) & 3]), "v"(b[(r + i) & 3]));
                if (OP == MFMA_FMA1 || OP == MFMA_FMA2)
                    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(va[i]) : "v"(x), "v"(x));
                if (OP == MFMA_FMA2)
                    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(va[(i + 3) & 7]) : "v"(x), "v"(x));
                if (OP == LDS_R32) asm volatile("ds_read_b32 %0, %1" : "=v"(v1) : "v"(t * 4));
                if (OP == LDS_R64) asm volatile("ds_read_b64 %0, %1" : "=v"(v2) : "v"(t * 8));
                if (OP == LDS_R128) asm volatile("ds_read_b128 %0, %1" : "=v"(v4) : "v"(t * 16));
                if (OP == LDS_W32) asm volatile("ds_write_b32 %0, %1" : : "v"(t * 4), "v"(v1));
                if (OP == LDS_W64) asm volatile("ds_write_b64 %0, %1" : : "v"(t * 8), "v"(v2));
                if (OP == LDS_W128) asm volatile("ds_write_b128 %0, %1" : : "v"(t * 16), "v"(v4));
            }
            asm volatile("s_waitcnt lgkmcnt(0)");
        }
    }
    float s = (float)(v4[0] + v4[3] + v2[0] + v2[1] + v1);
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + va[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

struct Bench {
    float *out;
    unsigned *w;
    int cus;
    double ghz;
    bool first = true;

    template <int OP> void run(const char *name, int wg_per_cu)
    {
        const int iters = 1000, nblk = cus * wg_per_cu;
        hipEvent_t a, b;
        (void)hipEventCreate(&a);
        (void)hipEventCreate(&b);
        probe<OP><<<nblk, 256>>>(out, w, 10);
        (void)hipDeviceSynchronize();
        (void)hipEventRecord(a);
        probe<OP><<<nblk, 256>>>(out, w, iters);
        (void)hipEventRecord(b);
        (void)hipEventSynchronize(b);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, a, b);
        (void)hipEventDestroy(a);
        (void)hipEventDestroy(b);
        // wavefront instructions of the probed form per SIMD (4 SIMDs per CU, 4 wavefronts per workgroup)
        const double per_simd = (double)wg_per_cu * iters * 8 * 16;
        std::printf("%s\n    {\"op\": \"%s\", \"wavefronts_per_simd\": %d, \"ms\": %.4f, \"clocks_per_instruction\": %.3f}",
                    first ? "" : ",", name, wg_per_cu, ms, ms * 1e-3 * ghz * 1e9 / per_simd);
        first = false;
    }

    template <int OP> void run2(const char *name, int wg_per_cu)
    {
        const int iters = 1000, nblk = cus * wg_per_cu;
        hipEvent_t a, b;
        (void)hipEventCreate(&a);
        (void)hipEventCreate(&b);
        probe2<OP><<<nblk, 256>>>(out, w, 10);
        (void)hipDeviceSynchronize();
        (void)hipEventRecord(a);
        probe2<OP><<<nblk, 256>>>(out, w, iters);
        (void)hipEventRecord(b);
        (void)hipEventSynchronize(b);
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, a, b);
        (void)hipEventDestroy(a);
        (void)hipEventDestroy(b);
        const double per_simd = (double)wg_per_cu * iters * 4 * 8;
        std::printf(",\n    {\"op\": \"%s\", \"wavefronts_per_simd\": %d, \"ms\": %.4f, \"clocks_per_instruction\": %.3f}",
                    name, wg_per_cu, ms, ms * 1e-3 * ghz * 1e9 / per_simd);
    }
};

}  // namespace

int main()
{
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) {
        std::fprintf(stderr, "valu_probe: no HIP device\n");
        return 2;
    }
    Bench b;
    b.cus = prop.multiProcessorCount;
    b.ghz = prop.clockRate * 1e-6;   // kHz -> GHz (peak engine clock)
    if (hipMalloc(&b.out, (size_t)b.cus * 4 * 256 * sizeof(float)) != hipSuccess ||
        hipMalloc(&b.w, 64) != hipSuccess || hipMemset(b.w, 0x3f, 64) != hipSuccess)
        return 2;
    std::printf("{\"device\": \"%s\", \"compute_units\": %d, \"clock_GHz\": %.3f, \"rows\": [", prop.name, b.cus, b.ghz);
    for (int wg = 1; wg <= 4; wg *= 2) {
        b.run<DOT2_SGPR>("v_dot2c_f32_bf16 (scalar multiplicand)", wg);
        b.run<FMAC_SGPR>("v_fmac_f32 (scalar multiplicand)", wg);
        b.run<FMAC_VGPR>("v_fmac_f32 (vector operands)", wg);
    }
    b.run<DOT2_VGPR>("v_dot2c_f32_bf16 (vector operands)", 4);
    b.run<MUL_VGPR>("v_mul_f32", 4);
    b.run<ADD_VGPR>("v_add_f32", 4);
    b.run<MAX_VGPR>("v_max_f32", 4);
    b.run<CVT_PK_BF16>("v_cvt_pk_bf16_f32", 4);
    b.run<AND_VGPR>("v_and_b32", 4);
    b.run<LSHL16>("v_lshlrev_b32", 4);
    b.run<PERM>("v_perm_b32", 4);
    b.run<MOV_SGPR>("v_mov_b32 from scalar", 4);
    b.run<READLANE>("v_readlane_b32", 4);
    for (int wg = 2; wg <= 4; wg *= 2) {
        b.run<MIX_NONE>("dot2c stream", wg);
        b.run<MIX_SMOV>("dot2c stream + s_mov_b32 per 4 (clocks per dot2c)", wg);
        b.run<MIX_WAITCNT>("dot2c stream + s_waitcnt per 4 (clocks per dot2c)", wg);
        b.run<MIX_LDS>("dot2c stream + ds_read_b32 per 4 (clocks per dot2c)", wg);
        b.run<MIX_READLANE>("dot2c stream + v_readlane_b32 per 4 (clocks per dot2c)", wg);
    }
    for (int wg = 2; wg <= 4; wg *= 2) {
        b.run2<MFMA>("v_mfma_f32_4x4x4_16b_bf16", wg);
        b.run2<MFMA_FMA1>("v_mfma_f32_4x4x4_16b_bf16 + 1 v_fmac_f32 (clocks per pair)", wg);
        b.run2<MFMA_FMA2>("v_mfma_f32_4x4x4_16b_bf16 + 2 v_fmac_f32 (clocks per triple)", wg);
    }
    b.run2<LDS_R32>("ds_read_b32", 4);
    b.run2<LDS_R64>("ds_read_b64", 4);
    b.run2<LDS_R128>("ds_read_b128", 4);
    b.run2<LDS_W32>("ds_write_b32", 4);
    b.run2<LDS_W64>("ds_write_b64", 4);
    b.run2<LDS_W128>("ds_write_b128", 4);
    std::printf("\n]}\n");
    (void)hipDeviceSynchronize();
    (void)hipFree(b.out);
    (void)hipFree(b.w);
    return 0;
}
