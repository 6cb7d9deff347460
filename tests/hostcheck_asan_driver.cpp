// Memory-safety driver of the host build: every buffer is heap-allocated at its exact size,
// so AddressSanitizer reports any global access the kernels make outside a tensor.  Built and
// run by tests/test_hostcheck_asan.py:
//   g++ -fsanitize=address,undefined -g -O1 tests/hostcheck_asan_driver.cpp -o <tmp>/driver
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../deconver_amd/csrc/ndc_hostcheck.cpp"

struct Case {
    int B, G, m, sc, D, H, W, kD, kH, kW, dtype, path;
};

static int run_case(const Case &c)
{
    ndc_geom g;
    g.batch = c.B;
    g.groups = c.G;
    g.m = c.m;
    g.sc = c.sc;
    g.size[0] = c.D;
    g.size[1] = c.H;
    g.size[2] = c.W;
    g.kernel[0] = c.kD;
    g.kernel[1] = c.kH;
    g.kernel[2] = c.kW;
    g.dtype = c.dtype;
    g.relu_input = 1;
    g.path = c.path;
    g.eps = 1e-16f;
    const size_t esz = c.dtype == NDC_BF16 ? 2 : 4;
    const size_t sp = (size_t)c.D * c.H * c.W;
    const size_t nx = (size_t)c.B * c.G * c.m * sp, ns = (size_t)c.B * c.G * c.sc * sp;
    const size_t nh = (size_t)c.G * c.m * c.sc * c.kD * c.kH * c.kW;
    auto fill = [&](size_t n) {
        unsigned char *p = (unsigned char *)malloc(n * esz);
        for (size_t i = 0; i < n; ++i) {
            float v = (float)((i * 2654435761u) % 1000) / 1000.0f;
            if (esz == 4) ((float *)p)[i] = v;
            else ((unsigned short *)p)[i] = ndc::float_to_bf16(v);
        }
        return p;
    };
    unsigned char *x = fill(nx), *z = fill(ns), *gout = fill(ns);
    unsigned char *out = (unsigned char *)malloc(ns * esz), *t1 = (unsigned char *)malloc(nx * esz);
    unsigned char *gx = (unsigned char *)malloc(nx * esz), *gz = (unsigned char *)malloc(ns * esz);
    unsigned char *inv = (unsigned char *)malloc(ns * esz), *rat = (unsigned char *)malloc(ns * esz);
    std::vector<float> h(nh, 0.05f), bias((size_t)c.G * c.sc, 0.1f), gh(nh), gb((size_t)c.G * c.sc);
    const size_t fws = ndc_forward_workspace_bytes(&g);
    void *fw = nullptr;
    if (posix_memalign(&fw, 256, fws ? fws : 256)) return -100;
    int st = ndc_forward(&g, x, z, h.data(), bias.data(), out, t1, inv, rat, fw, fws, nullptr);
    free(fw);
    if (st) return st;
    const size_t wsb = ndc_backward_workspace_bytes(&g, 1, 1, 1, 1);
    void *ws = nullptr;
    if (posix_memalign(&ws, 256, wsb ? wsb : 256)) return -100;
    // once re-gathering the denominator and ratio, once with the forward's copies
    st = ndc_backward(&g, x, z, t1, nullptr, nullptr, h.data(), bias.data(), gout, gx, gz,
                      gh.data(), gb.data(), ws, wsb, nullptr);
    if (!st)
        st = ndc_backward(&g, x, z, t1, inv, rat, h.data(), bias.data(), gout, gx, gz, gh.data(),
                          gb.data(), ws, wsb, nullptr);
    free(ws);
    free(x); free(z); free(gout); free(out); free(t1); free(gx); free(gz); free(inv); free(rat);
    return st;
}

// The block-level entry points on exactly sized buffers (rows cut into several parts, a ragged
// last part, a row length that is not a whole number of 16-byte vectors).
static int run_block_level(int dtype)
{
    const int esz = dtype == NDC_BF16 ? 2 : 4;
    const long long B = 2, C = 3, n = 2 * 8192 + 2048 + 5, rows = B * C;
    const size_t bytes = (size_t)(rows * n * esz);
    void *x = calloc(1, bytes), *y = malloc(bytes), *g = calloc(1, bytes), *gx = malloc(bytes);
    float *stats = (float *)malloc(sizeof(float) * 2 * rows);
    float bias[3] = {0.1f, -0.2f, 0.3f};
    const size_t wsb = ndc_rownorm_workspace_bytes(rows, n);
    void *ws = malloc(wsb);
    const long long parts = ndc_bias_act_parts(rows, n);
    float *gpart = (float *)malloc(sizeof(float) * rows * parts);
    int st = ndc_rownorm_forward(x, y, stats, rows, n, dtype, 1e-5f, ws, wsb, nullptr);
    if (!st) st = ndc_rownorm_backward(g, y, stats, x, gx, rows, n, dtype, ws, wsb, nullptr);
    if (!st) st = ndc_bias_act(x, bias, g, y, B, C, n, NDC_ACT_GELU, dtype, nullptr);
    if (!st) st = ndc_bias_act_backward(g, x, bias, gx, gpart, B, C, n, NDC_ACT_GELU, dtype, nullptr);
    if (!st) st = ndc_row_sums(g, gpart, rows, n, dtype, nullptr);
    if (!st) st = ndc_relayout(x, y, B, C, n, dtype, 1, nullptr);
    {
        float *cstats = (float *)malloc(sizeof(float) * 2 * B * n);
        const long long cparts = ndc_chnorm_parts(B, n, dtype);
        float *cpart = (float *)malloc(sizeof(float) * cparts * C * 2);
        if (!st) st = ndc_chnorm_forward(x, bias, bias, y, cstats, B, C, n, dtype, 1e-5f, nullptr);
        if (!st) st = ndc_chnorm_backward(g, x, cstats, bias, gx, cpart, B, C, n, dtype, nullptr);
        free(cstats); free(cpart);
    }
    free(gpart); free(ws); free(stats); free(x); free(y); free(g); free(gx);
    // 2 x 2 x 2 windows of a (rows, 4, 6, 16) grid and back
    const long long D = 4, H = 6, W = 16, m = rows * D * H * W;
    void *fine = calloc(1, (size_t)(m * esz)), *coarse = malloc((size_t)(m * esz)), *back = malloc((size_t)(m * esz));
    if (!st) st = ndc_regroup(fine, coarse, nullptr, rows, C, D, H, W, 1, dtype, 1, nullptr);
    if (!st) st = ndc_regroup(coarse, back, bias, rows, C, D, H, W, 1, dtype, 0, nullptr);
    free(fine); free(coarse); free(back);
    if (dtype == NDC_BF16) {
        // the streaming GEMM's host loops: 128 -> 64 channels of 2 x 128 voxels, every tail, the
        // transposed packing and the gradient mode with its rows of sums
        const long long cin = 128, cout = 64, nv = 128;
        void *px = calloc(1, (size_t)(B * cin * nv * 2)), *py = malloc((size_t)(B * cout * nv * 2));
        void *pz = malloc((size_t)(B * cout * nv * 2)), *pr = calloc(1, (size_t)(B * cout * nv * 2));
        void *pg = malloc((size_t)(B * cin * nv * 2));
        float *w = (float *)calloc((size_t)(cin * cout), sizeof(float)), *b64 = (float *)calloc((size_t)cout, sizeof(float));
        float *b128 = (float *)calloc((size_t)cin, sizeof(float));
        void *wf = aligned_alloc(16, ndc_pointwise_weight_bytes(cin, cout));
        void *wft = aligned_alloc(16, ndc_pointwise_weight_bytes(cout, cin));
        float *sums = (float *)malloc(sizeof(float) * (size_t)(ndc_pointwise_gemm_parts() * cin));
        if (!st) st = ndc_pointwise_gemm_supported(cin, cout, nv, dtype) ? 0 : -2;
        if (!st) st = ndc_pointwise_pack(w, NDC_F32, 0, wf, cin, cout, nullptr);
        if (!st) st = ndc_pointwise_pack(w, NDC_F32, 1, wft, cout, cin, nullptr);   // W^T from W as it lies
        if (!st) st = ndc_pointwise_gemm(px, wf, b64, pr, py, pz, B, cin, cout, nv, NDC_ACT_GELU, dtype, nullptr);
        if (!st) st = ndc_pointwise_gemm(px, wf, nullptr, nullptr, py, nullptr, B, cin, cout, nv, NDC_ACT_NONE, dtype, nullptr);
        if (!st) st = ndc_pointwise_gemm_actgrad(py, wft, b128, px, pg, sums, B, cout, cin, nv, NDC_ACT_GELU, dtype, nullptr);
        free(px); free(py); free(pz); free(pr); free(pg); free(w); free(b64); free(b128); free(wf); free(wft); free(sums);
    }
    printf("block-level entry points dtype%d -> status %d\n", dtype, st);
    return st;
}

int main()
{
    const Case cases[] = {
        {2, 3, 1, 4, 5, 9, 8, 3, 3, 3, NDC_F32, NDC_PATH_FUSED},
        {1, 1, 1, 4, 3, 16, 64, 3, 3, 3, NDC_BF16, NDC_PATH_FUSED},   // workgroups of four full wavefronts
        {1, 2, 1, 4, 2, 32, 32, 3, 3, 3, NDC_BF16, NDC_PATH_FUSED},
        {1, 2, 1, 4, 3, 7, 13, 3, 3, 3, NDC_BF16, NDC_PATH_FUSED},
        {1, 2, 1, 4, 6, 3, 70, 3, 3, 3, NDC_F32, NDC_PATH_FUSED},
        {1, 2, 1, 4, 5, 9, 8, 3, 3, 3, NDC_BF16, NDC_PATH_FUSED},
        {2, 1, 1, 4, 4, 5, 70, 3, 3, 3, NDC_BF16, NDC_PATH_FUSED},
        {1, 1, 1, 4, 1, 1, 1, 3, 3, 3, NDC_F32, NDC_PATH_FUSED},
        {2, 3, 1, 4, 1, 9, 12, 1, 5, 5, NDC_F32, NDC_PATH_FUSED},
        {1, 2, 1, 4, 1, 3, 70, 1, 5, 5, NDC_BF16, NDC_PATH_FUSED},
        {2, 2, 1, 4, 1, 7, 9, 1, 3, 3, NDC_F32, NDC_PATH_FUSED},
        {1, 2, 1, 4, 2, 40, 33, 3, 3, 3, NDC_F32, NDC_PATH_FUSED},
        {2, 3, 2, 2, 5, 4, 3, 3, 3, 3, NDC_F32, NDC_PATH_DIRECT},
        {1, 2, 3, 2, 1, 6, 5, 1, 3, 5, NDC_BF16, NDC_PATH_DIRECT},
    };
    int bad = 0;
    for (const Case &c : cases) {
        const int st = run_case(c);
        char first[256];
        const long long faults = ndc_host_faults(first, sizeof first);
        printf("case B%d G%d m%d sc%d %dx%dx%d k%dx%dx%d dtype%d path%d -> status %d, lds faults %lld %s\n",
               c.B, c.G, c.m, c.sc, c.D, c.H, c.W, c.kD, c.kH, c.kW, c.dtype, c.path, st, faults, first);
        if (st || faults) ++bad;
    }
    if (run_block_level(NDC_F32)) ++bad;
    if (run_block_level(NDC_BF16)) ++bad;
    return bad ? 1 : 0;
}
