/*
 * deconver_ndc.h -- C ABI of the MI355X (gfx950) implementation of Deconver's
 * nonnegative-deconvolution (NDC) source update.
 *
 * One call = one multiplicative update of the source, or its gradients:
 *
 *     s   = relu_input ? max(z + bias, 0) : z (+ bias)
 *     t1  = K(s)                                  K(u)[o,p] = sum_{i,tau} u[i,p+tau-pad] h[o,i,tau]
 *     out = s * (A(x) + eps) / (A(t1) + eps)      A(v)[i,p] = sum_{o,tau} v[o,p+pad-tau] h[o,i,tau]
 *
 * Conventions shared by every entry point
 *   - plain pointers to DEVICE memory, sizes in the geometry struct, a hipStream_t passed
 *     as void*; no framework types.  The caller owns every buffer (inputs, outputs,
 *     workspace); the library never allocates, frees or retains pointers.
 *   - launches are asynchronous on `stream`; nothing synchronises the host.
 *   - return value: 0 on success, a negative ndc_status otherwise; nothing throws.
 *   - layouts: x, t1, gx are (B, G*m, D, H, W); z, out, gout, gz are (B, G*sc, D, H, W),
 *     contiguous, channel g*sc+i = group g, source i; h, gh are (G, m, sc, kD, kH, kW)
 *     float32; bias, gb are (G*sc) float32.  Rank-1/2 problems use leading extents of 1
 *     (size = {1,1,W} / {1,H,W}, kernel likewise).  Stride 1, zero padding k/2, odd k.
 *   - dtype tags the storage of the activation tensors only; arithmetic and the
 *     filter/bias and their gradients are float32.
 */
#ifndef DECONVER_NDC_H
#define DECONVER_NDC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum ndc_dtype { NDC_F32 = 0, NDC_BF16 = 1 };

enum ndc_status {
    NDC_OK = 0,
    NDC_ERR_NULL = -1,        /* a required pointer is null */
    NDC_ERR_GEOMETRY = -2,    /* extents/kernel/groups outside what the kernels cover */
    NDC_ERR_DTYPE = -3,       /* unknown dtype tag */
    NDC_ERR_WORKSPACE = -4,   /* workspace too small or misaligned */
    NDC_ERR_LAUNCH = -5,      /* hipGetLastError() reported a failure after a launch */
    NDC_ERR_SCRATCH_LIMIT = -6 /* ndc_forward_noalloc: the geometry needs more scratch than
                                  NDC_NOALLOC_SCRATCH_BYTES */
};

/* Which implementation a call may use.  AUTO picks the fused LDS-tiled kernels when the
 * geometry is one they cover and the direct kernels otherwise; FUSED insists on the fused
 * kernels.  For both, the kernel FAMILY of bfloat16 3x3x3 calls is the process default
 * (ndc_matrix_kernels).  FUSED_VECTOR and FUSED_MATRIX are FUSED with the family named by
 * the call itself: tap sums on the vector unit (v_dot2c_f32_bf16), or on the 4x4x4 matrix
 * instruction where those kernels cover the geometry (row widths 8, 16, 32, 64, 128; the
 * vector-unit kernels elsewhere).  A call that names its family reads no process-wide state,
 * so a forward call on one thread and its backward call on another (an autograd engine
 * thread) cannot disagree, whatever a third thread does to the default. */
enum ndc_path {
    NDC_PATH_AUTO = 0,
    NDC_PATH_DIRECT = 1,
    NDC_PATH_FUSED = 2,
    NDC_PATH_FUSED_MATRIX = 3,
    NDC_PATH_FUSED_VECTOR = 4
};

typedef struct ndc_geom {
    int32_t batch;       /* B */
    int32_t groups;      /* G */
    int32_t m;           /* filter channels per group, C = G*m */
    int32_t sc;          /* source channels per group */
    int32_t size[3];     /* D, H, W */
    int32_t kernel[3];   /* kD, kH, kW (odd) */
    int32_t dtype;       /* ndc_dtype of x, z, out, t1, gout, gx, gz */
    int32_t relu_input;  /* 1: s = max(z + bias, 0); 0: s = z + bias (bias usually null) */
    int32_t path;        /* ndc_path */
    float eps;
} ndc_geom;

/* Library version (major*10000 + minor*100 + patch). */
int ndc_version(void);

/* Human-readable text for a status code (static storage). */
const char *ndc_status_string(int status);

/* 1 if the fused LDS-tiled kernels cover `g`, else 0.
 * Counterpart of kernels_supported()/fused_kernels_apply()
 * (deconver/deconvolution/kernels.py:143-163, functional.py:34-47). */
int ndc_fused_supported(const ndc_geom *g);

/* 0 if some path covers `g` (then every entry point below accepts it), else a status. */
int ndc_check_geometry(const ndc_geom *g);

/* 1 if `ndc_backward` for `g` reads the forward's s_over_den / ratio when they are passed (so
 * that keeping them pays), 0 if its kernels re-gather regardless.  No counterpart in the
 * reference. */
int ndc_backward_uses_saved(const ndc_geom *g);

/* Process-wide DEFAULT of the kernel family, used by calls whose ndc_geom.path is AUTO or
 * FUSED (calls with FUSED_VECTOR / FUSED_MATRIX ignore it): on = 1 lets them run the bfloat16
 * 3x3x3 kernels that do their tap sums on the 4x4x4 matrix instruction (row widths 8, 16, 32,
 * 64, 128), on = 0 keeps them on the vector unit (v_dot2c_f32_bf16), on < 0 only queries;
 * returns the setting in force.  Default 0: the path is specified as a stencil without matrix
 * instructions, and the default build measures that; the other family is the faster one on
 * MI355X and gives the same results to the bf16 tolerance.  The setting is an atomic integer
 * read once per call; it is the only state the library keeps between calls (besides the
 * scratch array of ndc_forward_noalloc).  No counterpart in the reference. */
int ndc_matrix_kernels(int on);

/* Bytes of scratch `ndc_forward` needs for `g` (0 for most geometries; the bfloat16 3x3x3
 * kernels keep their packed filter tables there).  No counterpart in the reference, whose
 * wrappers allocate their own temporaries (kernels.py:728-788). */
size_t ndc_forward_workspace_bytes(const ndc_geom *g);

/*
 * Forward update.  Replaces DeconvUpdate.forward
 * (deconver/deconvolution/functional.py:105-116), i.e. the pair
 * kernels.gconv(z, K, relu, bias) + kernels.deconv_fwd(...)
 * (deconver/deconvolution/kernels.py:728-788).
 *   x, z, h       inputs;  bias may be null
 *   out           output, same shape/dtype as z
 *   t1            optional output K(s), same shape/dtype as x: pass it when a backward
 *                 call will follow (it is what the reference saves for backward), null
 *                 for inference
 *   s_over_den,   optional outputs s/(A(t1)+eps) and (A(x)+eps)/(A(t1)+eps), same
 *   ratio         shape/dtype as out; both or neither.  Handing them to ndc_backward lets it
 *                 skip re-gathering A(x) and A(t1): more memory kept between the two calls
 *                 (two tensors of the size of out) for fewer multiplications.  The
 *                 reference has no counterpart (it re-gathers, kernels.py:806-809).
 *   workspace     >= ndc_forward_workspace_bytes(g) bytes, 256-byte aligned (may be null
 *                 when that is 0)
 */
int ndc_forward(const ndc_geom *g, const void *x, const void *z, const float *h,
                const float *bias, void *out, void *t1, void *s_over_den, void *ratio,
                void *workspace, size_t workspace_bytes, void *stream);

/* Size of the device array behind ndc_forward_noalloc: room for the packed filter tables of
 * 824 depthwise channels (1272 bytes per channel). */
#define NDC_NOALLOC_SCRATCH_BYTES (1u << 20)

/*
 * ndc_forward without a workspace argument and without any allocation: same inputs, outputs
 * and results as ndc_forward, with the forward's scratch in a device array that is part of
 * the library image (each GPU the library runs on holds NDC_NOALLOC_SCRATCH_BYTES of it
 * until the process ends).  It has no counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  A geometry whose ndc_forward_workspace_bytes() exceeds the array is refused
 * with NDC_ERR_SCRATCH_LIMIT before anything is launched.  All calls on one GPU share the one
 * array: calls that may overlap on a GPU (different streams, different threads) race on it
 * and must be serialised by the caller, or use ndc_forward with a workspace of their own.
 * The array's device address is looked up once per device (hipGetSymbolAddress, no
 * allocation), for the device that is current when the call is made, which must be the
 * stream's device: by ndc_noalloc_init, or else by the first ndc_forward_noalloc call on that
 * device.  That lookup is not a stream operation and may be refused while a stream capture is
 * in progress, so a caller that captures calls ndc_noalloc_init (or makes one call) on each
 * device beforehand; every later call only launches kernels on `stream`.
 */
int ndc_forward_noalloc(const ndc_geom *g, const void *x, const void *z, const float *h,
                        const float *bias, void *out, void *t1, void *s_over_den, void *ratio,
                        void *stream);

/* Set-up of ndc_forward_noalloc for the current device (see above): looks up the scratch
 * array's address there.  Allocates nothing, launches nothing; 0 or a negative ndc_status.
 * Optional outside stream capture, idempotent, thread-safe.  No counterpart in the reference. */
int ndc_noalloc_init(void);

/*
 * Prepared filter tables.  Some kernel families read the filter from a packed table instead
 * of `h` (today: the bfloat16 3x3x3 kernels, 1272 bytes per channel).  ndc_forward and
 * ndc_backward pack it into their workspace on every call; a caller that runs several calls
 * with one filter (forward and backward of one step, several iterations of one layer) can
 * pack it once with ndc_prepare_taps and hand it to ndc_forward_taps / ndc_backward_taps,
 * which then launch nothing but the update kernels.  The table is a function of `h` and of
 * the filter geometry, channel count and dtype in `g` only (not of batch, extents, eps,
 * relu_input).  The reference keeps no such table (its kernels read h, kernels.py:728-894).
 *   ndc_taps_bytes     bytes of the table for `g`; 0 when the kernels for `g` read `h`
 *                      (then `taps` is ignored everywhere and may be null)
 *   ndc_prepare_taps   fills `taps` (256-byte aligned, >= ndc_taps_bytes(g)) from `h`
 *   ndc_forward_taps   ndc_forward with the table in place of the workspace
 *   ndc_backward_taps  ndc_backward with the table; workspace as for ndc_backward
 */
size_t ndc_taps_bytes(const ndc_geom *g);
int ndc_prepare_taps(const ndc_geom *g, const float *h, void *taps, size_t taps_bytes,
                     void *stream);
int ndc_forward_taps(const ndc_geom *g, const void *x, const void *z, const float *h,
                     const void *taps, const float *bias, void *out, void *t1, void *s_over_den,
                     void *ratio, void *stream);
int ndc_backward_taps(const ndc_geom *g, const void *x, const void *z, const void *t1,
                      const void *s_over_den, const void *ratio, const float *h, const void *taps,
                      const float *bias, const void *gout, void *gx, void *gz, float *gh, float *gb,
                      void *workspace, size_t workspace_bytes, void *stream);

/* Bytes of scratch `ndc_backward` needs for `g` with the requested outputs (each flag
 * nonzero when the matching output pointer will be non-null). */
size_t ndc_backward_workspace_bytes(const ndc_geom *g, int need_gx, int need_gz, int need_gh,
                                    int need_gb);

/*
 * Backward of the update.  Replaces DeconvUpdate.backward
 * (deconver/deconvolution/functional.py:118-182), i.e. kernels.deconv_bwd, gconv x2,
 * wgrad x3, deconv_gz and the bias reduction (kernels.py:791-894).
 *   x, z, t1, h, bias   what the forward call saw / produced (bias may be null)
 *   s_over_den, ratio   what the forward call wrote for the same inputs, or both null (then
 *                       the kernels re-gather A(x) and A(t1)); results agree to rounding
 *   gout                upstream gradient, shape/dtype of out
 *   gx, gz, gh, gb      optional outputs (null = not needed); gh and gb are OVERWRITTEN,
 *                       not accumulated into.  gx is only the NDC term K(gn); the
 *                       projection's own input gradient is the caller's business.
 *   workspace           >= ndc_backward_workspace_bytes(...) bytes, 256-byte aligned
 */
int ndc_backward(const ndc_geom *g, const void *x, const void *z, const void *t1,
                 const void *s_over_den, const void *ratio, const float *h, const float *bias,
                 const void *gout, void *gx, void *gz, float *gh, float *gb, void *workspace,
                 size_t workspace_bytes, void *stream);

/*
 * ndc_backward with a stopwatch: same arguments and results, plus pass_ms[3] = device time in
 * milliseconds of (pass 1: gn/gd, gx, gt1, A-side filter terms), (pass 2: gz, gb, K-side
 * filter term) and (the partial-sum reduction), taken with events on `stream`.  The call
 * synchronises the host with `stream`.  Measurement aid for the benchmark harness; it has no
 * counterpart in the reference (its benchmarks time whole calls, benchmarks/bench_deconv.py:109-121).
 * The direct path is not instrumented and reports zeros.
 */
int ndc_backward_profiled(const ndc_geom *g, const void *x, const void *z, const void *t1,
                          const void *s_over_den, const void *ratio, const float *h,
                          const float *bias, const void *gout, void *gx, void *gz, float *gh,
                          float *gb, void *workspace, size_t workspace_bytes, void *stream,
                          float *pass_ms);

/*
 * Plain grouped convolution with the same tap conventions (adjoint = 0: K, 1: A), input
 * and output in g->dtype; optional on-load bias + ReLU of the input as in the forward.
 * Replaces kernels.gconv (deconver/deconvolution/kernels.py:728-759).  The update entry points
 * above do not call it (they apply K and A inside their own kernels); it is exported for
 * callers and tests that need K or A alone.  Runs the direct kernels for every geometry.
 */
int ndc_gconv(const ndc_geom *g, const void *in, const float *h, const float *bias, int adjoint,
              void *out, void *stream);

/*
 * Channels-last entry.  The update kernels read channel-first tensors (B, C, D, H, W): all 64
 * lanes of a wavefront then work on one channel, whose filter taps are wave-uniform and sit in
 * scalar registers.  A caller that holds its activations channels-last (B, D, H, W, C in
 * memory: torch.channels_last / channels_last_3d) brings them in, and takes results out,
 * through this copy: an LDS-tiled transposition that runs near the device-copy bandwidth,
 * where a generic strided copy takes 4 to 18 times as long (measured on MI355X, bfloat16:
 * the 512-channel source tensor of config 3, and the 2 GiB source tensor of a 64-channel
 * 128^3 layer).
 *   src, dst           distinct device buffers of batch * channels * spatial elements
 *   spatial            D * H * W
 *   dtype              ndc_dtype of the elements
 *   to_channels_last   0: src is channels-last (B, S, C), dst becomes channel-first (B, C, S);
 *                      1: the reverse
 * The reference's fused path accepts contiguous channel-first tensors only and copies
 * anything else first (deconver/deconvolution/kernels.py:118-127, deconv.py:155).
 */
int ndc_relayout(const void *src, void *dst, int64_t batch, int64_t channels, int64_t spatial,
                 int dtype, int to_channels_last, void *stream);

/*
 * Row normalisation: y = (x - mean) / sqrt(var + eps) over each of `rows` contiguous rows of n
 * elements (biased variance, float32 statistics), and its gradient.  On a channel-first tensor
 * (B, C, *S) with rows = B * C and n = prod(S) this is InstanceNorm without affine parameters
 * or running statistics: the norm1 / norm2 of a Deconver block (deconver/deconver.py:52-64) in
 * the 2-D and 3-D segmentation networks, i.e. the producer of every NDC layer's input and the
 * consumer of its gradient.  A row of the 3-D network's first level is 128^3 elements long and
 * there are 128 of them, so each row is cut over many workgroups (two launches per direction:
 * partial sums, then the transform).  HBM traffic: 2 reads + 1 write of the tensor forward,
 * 4 reads + 1 write backward.
 *   x, y         distinct device buffers of rows * n elements of `dtype`
 *   stats        rows * 2 floats: (mean, 1/sqrt(var + eps)) per row; written by the forward,
 *                read by the backward
 *   gy, gx       gradient of y (in), of x (out); gx may be gy
 *   addend       NULL, or a tensor like gy that is added to gx: the gradient that reaches x
 *                around the norm (the residual branch of a pre-norm block,
 *                deconver/deconver.py:63-64), which otherwise costs a pass of its own; gx may
 *                be addend
 *   workspace    ndc_rownorm_workspace_bytes(rows, n) bytes of device memory, 8-byte aligned;
 *                contents need not survive between calls
 * The backward takes the forward's OUTPUT y (the normalised rows), not x.
 */
size_t ndc_rownorm_workspace_bytes(int64_t rows, int64_t n);
int ndc_rownorm_forward(const void *x, void *y, float *stats, int64_t rows, int64_t n, int dtype,
                        float eps, void *workspace, size_t workspace_bytes, void *stream);
int ndc_rownorm_backward(const void *gy, const void *y, const float *stats, const void *addend, void *gx,
                         int64_t rows, int64_t n, int dtype, void *workspace, size_t workspace_bytes,
                         void *stream);

/*
 * What follows a 1x1 projection in a Deconver block, in one pass over the projection's output:
 *   y[b][c][i] = act(z[b][c][i] + bias[c]) + residual[b][c][i]
 * on channel-first tensors of batch * channels rows of n elements.  It stands for the bias of
 * the mixer's out_proj and of the MLP's two projections, the MLP's GELU and the block's
 * residual sums (deconver/deconver.py:41-46, 60-64; deconver/layers/mlp.py:40-63), which
 * PyTorch runs as separate passes over the tensor.
 *   bias       `channels` floats, or NULL
 *   residual   a tensor like z, or NULL
 *   y          may be z (in place)
 *   act        ndc_act; the GELU is the exact one, u * Phi(u)
 * ndc_bias_act_backward: gz = gy * act'(z + bias) for NDC_ACT_RELU / NDC_ACT_GELU (gz may be
 * gy), and, if gpart is not NULL, gpart[row * parts + p] = the sum of gz over part p of the
 * row, parts = ndc_bias_act_parts(batch * channels, n): the bias gradient is their sum over the
 * batch and the parts.  (With NDC_ACT_NONE the gradient of z is gy itself; the call is refused.)
 */
enum ndc_act { NDC_ACT_NONE = 0, NDC_ACT_RELU = 1, NDC_ACT_GELU = 2 };
/*
 * ndc_row_sums: partial[row * parts + p] = the sum of part p of row `row` of a (rows, n) matrix,
 * parts = ndc_bias_act_parts(rows, n), float32.  The bias gradient of a projection without
 * activation (nn.Conv1d's in deconver/layers/linear.py:53-58) is the sum of these over the
 * batch and the parts of its output gradient.
 */
int ndc_row_sums(const void *x, float *partial, int64_t rows, int64_t n, int dtype, void *stream);
int64_t ndc_bias_act_parts(int64_t rows, int64_t n);
int ndc_bias_act(const void *z, const float *bias, const void *residual, void *y, int64_t batch,
                 int64_t channels, int64_t n, int act, int dtype, void *stream);
int ndc_bias_act_backward(const void *gy, const void *z, const float *bias, void *gz, float *gpart,
                          int64_t batch, int64_t channels, int64_t n, int act, int dtype, void *stream);

/*
 * The 1x1 projection itself, with its tail, for bfloat16 channel-first tensors:
 *   y[b][co][i] = act( sum_ci W[co][ci] * x[b][ci][i] + bias[co] ) + residual[b][co][i]
 * (nn.Conv1d with kernel size 1 in deconver/layers/linear.py:53-58, followed by what
 * deconver/deconver.py:41-46, 60-64 and deconver/layers/mlp.py:40-63 apply to its output).
 * A streaming kernel on the matrix units: x is read once, y written once, float32 accumulation,
 * one rounding of the result.
 *   ndc_pointwise_gemm_supported  1 where the kernel applies: NDC_BF16; cin 64, 128 or 256, or a
 *                  larger multiple of 64 with cout <= 128; cout a multiple of 32;
 *                  cin * cout * 2 <= 128 KiB; n a multiple of 64; else 0 (callers then use a
 *                  library GEMM and ndc_bias_act)
 *   ndc_pointwise_pack  writes W in the order the kernel reads it into wfrag
 *                  (ndc_pointwise_weight_bytes(cin, cout) bytes, 16-byte aligned): the 8 values
 *                  W[32 c + l % 32][16 s + 8 (l / 32) + 0..7], as bf16, at element
 *                  (((c * cin / 16) + s) * 64 + l) * 8.  w: cout x cin row-major, float32 or
 *                  bf16; with transposed != 0 the same matrix stored as cin x cout (so that the
 *                  input gradient, W^T gy, packs the weight as it lies).
 *   x              (batch, cin, n); y, residual, zkeep: (batch, cout, n); all bf16, 4-byte aligned
 *   bias           cout floats or NULL; residual NULL or a tensor added to the result
 *   zkeep          NULL, or (with NDC_ACT_RELU / NDC_ACT_GELU) receives the product before bias
 *                  and activation (what ndc_bias_act_backward reads as z)
 * With more than 256 input channels (the projections back from a widened tensor) the call takes
 * NDC_ACT_NONE and no zkeep: product, bias and residual.
 */
int ndc_pointwise_gemm_supported(int64_t cin, int64_t cout, int64_t n, int dtype);
size_t ndc_pointwise_weight_bytes(int64_t cin, int64_t cout);
int ndc_pointwise_pack(const void *w, int w_dtype, int transposed, void *wfrag, int64_t cin, int64_t cout,
                       void *stream);
int ndc_pointwise_gemm(const void *x, const void *wfrag, const float *bias, const void *residual, void *y,
                       void *zkeep, int64_t batch, int64_t cin, int64_t cout, int64_t n, int act, int dtype,
                       void *stream);
/*
 * ndc_pointwise_gemm_masked: y = (W x + bias + residual) where mask > 0, else 0; mask of y's shape.
 * The input gradient of a projection whose input is a rectifier's output (mask), with another
 * gradient of the same tensor (residual) accumulated on the way: DeconvMixer's ReLU between
 * in_proj and the layer (deconver/deconver.py:29-46), whose backward is then no pass of its own.
 * Shapes and alignment as for ndc_pointwise_gemm; y may be residual.
 */
int ndc_pointwise_gemm_masked(const void *x, const void *wfrag, const float *bias, const void *residual,
                              const void *mask, void *y, int64_t batch, int64_t cin, int64_t cout, int64_t n,
                              int dtype, void *stream);
/*
 * The input gradient of a projection whose INPUT was act(z + bias) (the second projection of
 * the MLP, deconver/layers/mlp.py:40-63, whose input is the GELU of the first one's output),
 * taken through that activation in the same kernel:
 *   gz[b][co][i] = ( sum_ci W[co][ci] * gy[b][ci][i] ) * act'(z[b][co][i] + bias[co])
 * with wfrag the packed TRANSPOSE of the projection's weight (ndc_pointwise_pack with
 * transposed != 0), act NDC_ACT_RELU or NDC_ACT_GELU, shapes as for ndc_pointwise_gemm with
 * cin <= 256.
 *   gpart          NULL, or ndc_pointwise_gemm_parts() * cout floats: per-wavefront sums of gz
 *                  (unused rows are zeroed); the gradient of `bias` is the sum over the rows
 */
int64_t ndc_pointwise_gemm_parts(void);
int ndc_pointwise_gemm_actgrad(const void *gy, const void *wfrag, const float *bias, const void *z, void *gz,
                               float *gpart, int64_t batch, int64_t cin, int64_t cout, int64_t n, int act,
                               int dtype, void *stream);

/*
 * Normalisation over the CHANNEL axis of a channel-first tensor (batch, channels, n):
 *   y[b][c][i] = (x[b][c][i] - mean[b][i]) * rstd[b][i] * weight[c] + bias[c],
 * mean and biased variance over c.  The reference's LayerNorm (deconver/layers/norm.py:25-34:
 * nn.LayerNorm with the channel axis moved last and back), the default norm of its blocks and
 * stem (deconver/deconver.py:52, 103), on the layout the tensors already have: nothing is
 * transposed.
 *   weight, bias   `channels` floats each, or NULL (1 and 0)
 *   stats          batch * 2 * n floats: mean then rstd per voxel; written by the forward, read
 *                  by the backward
 *   partial        NULL, or ndc_chnorm_parts(batch, n, dtype) * channels * 2 floats: per part
 *                  and channel (sum of gy * xhat, sum of gy); the gradients of weight and bias
 *                  are the sums over the parts
 *   x, y / gy, gx  distinct buffers; gx may be gy.  16-byte aligned buffers take 16-byte
 *                  accesses when n is a multiple of 16 bytes of elements.
 */
int64_t ndc_chnorm_parts(int64_t batch, int64_t n, int dtype);
int ndc_chnorm_forward(const void *x, const float *weight, const float *bias, void *y, float *stats,
                       int64_t batch, int64_t channels, int64_t n, int dtype, float eps, void *stream);
int ndc_chnorm_backward(const void *gy, const void *x, const float *stats, const float *weight, void *gx,
                        float *partial, int64_t batch, int64_t channels, int64_t n, int dtype, void *stream);

/*
 * Regrouping of a grid by 2 x 2 (depth2 = 0) or 2 x 2 x 2 (depth2 = 1) windows: the data
 * movement of the reference's 2-tap, stride-2 resampling convolutions (nn.ConvNd(kernel_size=2,
 * stride=2), nn.ConvTransposeNd(kernel_size=2, stride=2), deconver/unet.py:36-60, 108-131) once
 * their arithmetic is the 1x1 projection.
 *   to_channels = 1:  dst[r][k][d][h][w] = src[r][2d + kd][2h + kh][2w + kw],  k = (kd, kh, kw)
 *   to_channels = 0:  dst[r][2d + kd][2h + kh][2w + kw] = src[r][k][d][h][w] + bias[r % channels]
 *   rows       batch * channels of the fine-grid tensor
 *   D, H, W    the fine grid (D = 1 for images); H, W (and D with depth2) even, W a multiple of
 *              16 bytes of elements; src, dst distinct and 16-byte aligned -- anything else is
 *              refused with NDC_ERR_GEOMETRY and the caller copies by other means
 *   bias       NULL, or `channels` floats added on the way to the grid (the transposed
 *              convolution's bias); not allowed with to_channels = 1
 */
int ndc_regroup(const void *src, void *dst, const float *bias, int64_t rows, int64_t channels, int64_t D,
                 int64_t H, int64_t W, int depth2, int dtype, int to_channels, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* DECONVER_NDC_H */
