/*
 * pet_hip.h -- C ABI of the MI355X (gfx950) execution backend for PET tensor
 * programs. Every entry point is extern "C", takes plain pointers and sizes,
 * returns 0 on success and a non-zero pet_hip_status otherwise (no exceptions,
 * no exit() across the boundary). Device pointers are caller-owned; no call
 * here copies between host and device except the explicit memcpy functions,
 * and none retains a caller pointer after it returns.
 *
 * Citations name the reference interface (thu-pacman/PET) that each entry
 * point replaces, as path:line.
 *
 * All tensors are fp32, row-major, contiguous.
 */
#ifndef PET_HIP_H
#define PET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PET_HIP_MAX_RANK 8

#if defined(__GNUC__)
#define PET_HIP_API __attribute__((visibility("default")))
#else
#define PET_HIP_API
#endif

/* Empty tensors. An empty batch (n, b or bs of 0, no rows) or an empty output is not an
 * error: the call launches nothing, returns PET_HIP_OK and does not look at the pointers,
 * which may then be NULL. The reference's loop nests do the same by not running
 * (src/Graph/operator.cc:94-158, 620-654). A matmul over an empty k axis writes the bias
 * (zeros without one), a pad around an empty tensor writes zeros. Negative extents, and a
 * zero where the operator's shape rule needs a positive number (channels, filters, filter
 * extents, strides), are PET_HIP_ERR_INVALID. */
typedef enum pet_hip_status {
    PET_HIP_OK = 0,
    PET_HIP_ERR_INVALID = 1,     /* bad argument / shape the op rejects (reference: compute() == nullptr) */
    PET_HIP_ERR_UNSUPPORTED = 2, /* valid but not implemented (reference: perf() == INFINITY) */
    PET_HIP_ERR_RUNTIME = 3,     /* a HIP call failed; see pet_hip_last_error() */
    PET_HIP_ERR_NOT_INIT = 4
} pet_hip_status;

/* Operator::ActType, include/operator.h:95-100, plus GELU (absent upstream). */
typedef enum pet_hip_act {
    PET_HIP_ACT_NONE = 0,
    PET_HIP_ACT_RELU = 1,
    PET_HIP_ACT_SIGMOID = 2,
    PET_HIP_ACT_TANH = 3,
    PET_HIP_ACT_GELU = 4
} pet_hip_act;

typedef enum pet_hip_eltwise_op {
    PET_HIP_ADD = 0, /* AddOp::compute, src/Graph/operator.cc:2983-3002 */
    PET_HIP_SUB = 1, /* SubOp::compute, src/Graph/operator.cc:3074-3090 */
    PET_HIP_MUL = 2, /* MulOp::compute, src/Graph/operator.cc:3157-3176 */
    PET_HIP_DIV = 3  /* DivOp, shape rule src/Graph/operator.cc:3306-3313; a / b (the
                        reference's CPU body at :3259 subtracts) */
} pet_hip_eltwise_op;

/* Flags of the *_ex contraction entry points: what a graph runtime fuses across
 * launches. No counterpart upstream, where cuDNN / cuBLAS calls stand alone. */
typedef enum pet_hip_call_flags {
    /* y already holds bias (or zeros): a launch that accumulates into y (see the
     * *_accumulates queries) skips its initialising launch (a residual, if any, is
     * added along with the partial sums); bias must still be passed. Other launches
     * overwrite y as usual. */
    PET_HIP_CALL_Y_INITIALISED = 1,
    /* act is ReLU and every reader of y applies it on load (the two flags below): a
     * launch that accumulates into y leaves the ReLU out; others apply it as usual,
     * which the readers' second ReLU does not change. */
    PET_HIP_CALL_DEFER_RELU = 2,
    PET_HIP_CALL_X_RELU = 4,   /* use max(x, 0) for x */
    PET_HIP_CALL_RES_RELU = 8, /* use max(residual, 0) for the residual */
    /* pet_hip_bmm_ex_f32 only. A holds one [m,k] (or [k,m]) matrix that every batch entry
     * multiplies: an Extend of the lhs along dim 0 in front of a BatchMatmul (PET's matmul
     * merge, src/Mutant/generator.cc:1495-1552) folded into the addressing. */
    PET_HIP_CALL_A_SHARED = 16,
    /* pet_hip_bmm_ex_f32 only. bias is [b, n], one vector per batch entry: the per-slab
     * bias Adds that follow the Split of a merged BatchMatmul. */
    PET_HIP_CALL_BIAS_PER_BATCH = 32
} pet_hip_call_flags;

/* Convolution algorithms, the counterpart of the cuDNN algorithm list ConvOp::perf
 * times (src/Graph/operator.cc:296-515): how the K loop of a tile is shared out.
 * PET_HIP_CONV_ALGO(a) goes into the flags of pet_hip_conv2d_ex_f32 / conv3d_ex.
 * 0: the library's cost model decides (what every other entry point does); 1-5: 1, 2, 4,
 * 8, 16 workgroups per tile (clamped to what the shape allows); 6: stream-K (when the
 * shape admits it, else the cost model's split); 7: the cost model's split, never
 * stream-K. Every algorithm computes the same sums; with more than one workgroup per
 * tile their order, and so the last bits, can differ. */
#define PET_HIP_CONV_ALGO_COUNT 8
#define PET_HIP_CONV_ALGO(a) (((unsigned)(a) & 0xffu) << 8)

/* One output of pet_hip_bias_fill_batch: y[o][c][i] = bias[c] (zeros when bias is NULL). */
typedef struct pet_hip_fill {
    float *y;
    const float *bias;
    size_t outer, ch, inner;
} pet_hip_fill;

/* Opaque handles (a hipStream_t / hipEvent_t / hipGraphExec_t underneath). */
typedef void *pet_hip_stream_t;
typedef void *pet_hip_event_t;
typedef void *pet_hip_graph_t;

/* ---- context --------------------------------------------------------------
 * Replaces the cudnnCreate / cublasCreate / cudaMalloc block of
 * PerfEngine::PerfEngine and PerfEngine::allocMem (include/perf_engine.h:41-45,
 * src/Graph/perf_engine.cc:31-56) and checkCudaError (include/common.h:30-38). */
PET_HIP_API int pet_hip_init(int device);
PET_HIP_API int pet_hip_shutdown(void);
PET_HIP_API const char *pet_hip_last_error(void);
/* name of the device's architecture ("gfx950") and number of compute units */
PET_HIP_API int pet_hip_device_info(char *arch, size_t arch_len, int *num_cu);
/* on != 0: contractions whose K loop is split over workgroups add their partial
 * sums in a fixed order (one launch, partial tiles in library scratch), so equal
 * inputs give bit-equal outputs from run to run. Off (the default) they use float
 * atomics, which is faster and exact only up to summation order. The reference
 * leaves this to the cuDNN algorithm it picks per convolution
 * (src/Graph/operator.cc:296-515 loops over the algorithms). Environment variable
 * PET_HIP_DETERMINISTIC=1 sets the initial value. */
PET_HIP_API int pet_hip_set_deterministic(int on);
/* *on receives the current setting (for callers that switch it for a while) */
PET_HIP_API int pet_hip_get_deterministic(int *on);

/* ---- memory (cudaMalloc / cudaMemcpy / cudaFree call sites,
 * src/Graph/perf_engine.cc:31-47, src/Graph/code_engine.cc:560-643) ---------- */
PET_HIP_API int pet_hip_malloc(void **dptr, size_t bytes);
PET_HIP_API int pet_hip_free(void *dptr);
PET_HIP_API int pet_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, pet_hip_stream_t s);
PET_HIP_API int pet_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, pet_hip_stream_t s);
PET_HIP_API int pet_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, pet_hip_stream_t s);
/* fills n floats with value through a kernel (safe under graph capture) */
PET_HIP_API int pet_hip_fill_f32(float *dst, float value, size_t n, pet_hip_stream_t s);
/* uniform [lo, hi) fill from a counter-based generator, replaces
 * curandGenerateUniform (src/Graph/perf_engine.cc:49-55, code_engine.cc:582) */
PET_HIP_API int pet_hip_rand_uniform_f32(float *dst, size_t n, uint64_t seed, float lo, float hi,
                             pet_hip_stream_t s);

/* ---- streams, events, graphs ---------------------------------------------
 * Replace cudaDeviceSynchronize + std::chrono timing in Operator::perf
 * (src/Graph/operator.cc:416-467) and the cudaEvent bracket of the emitted
 * program (src/Graph/code_engine.cc:180-217). */
PET_HIP_API int pet_hip_stream_create(pet_hip_stream_t *s);
PET_HIP_API int pet_hip_stream_destroy(pet_hip_stream_t s);
PET_HIP_API int pet_hip_stream_sync(pet_hip_stream_t s);
PET_HIP_API int pet_hip_event_create(pet_hip_event_t *e);
PET_HIP_API int pet_hip_event_destroy(pet_hip_event_t e);
PET_HIP_API int pet_hip_event_record(pet_hip_event_t e, pet_hip_stream_t s);
PET_HIP_API int pet_hip_event_sync(pet_hip_event_t e);
PET_HIP_API int pet_hip_event_elapsed_ms(float *ms, pet_hip_event_t start, pet_hip_event_t stop);
/* Capture every launch issued on `s` between begin and end into an executable
 * graph; replaces the per-iteration op list of the emitted main()
 * (src/Graph/code_engine.cc:194-215). */
PET_HIP_API int pet_hip_graph_begin_capture(pet_hip_stream_t s);
PET_HIP_API int pet_hip_graph_end_capture(pet_hip_stream_t s, pet_hip_graph_t *g);
PET_HIP_API int pet_hip_graph_launch(pet_hip_graph_t g, pet_hip_stream_t s);
PET_HIP_API int pet_hip_graph_destroy(pet_hip_graph_t g);

/* ---- contractions ---------------------------------------------------------*/

/* ConvOp::computeShape with explicit padding, src/Graph/operator.cc:219-221:
 * o = (i - (k - s) * d + 2 p) / s. */
PET_HIP_API int pet_hip_conv_out_dim(int i, int k, int p, int s, int d);

/* Conv2d, NCHW x [n,c,h,w], weight [f, c/groups, r, s], y [n,f,oh,ow] with
 * oh/ow from pet_hip_conv_out_dim. Cross-correlation, zero padding, group of
 * output channel ff is ff / (f / groups). bias (may be NULL) is [f]; act is a
 * pet_hip_act. Semantics: ConvOp::compute, src/Graph/operator.cc:94-158;
 * replaces cudnnConvolutionForward / cudnnConvolutionBiasActivationForward
 * (src/Graph/operator.cc:425-427, 478-481; src/Graph/code_engine.cc:869-977).
 * Returns PET_HIP_ERR_INVALID when c % (c/groups) or f % groups != 0. */
PET_HIP_API int pet_hip_conv2d_f32(const float *x, const float *w, const float *bias, float *y,
                       int n, int c, int h, int wd, int f, int r, int s, int ph, int pw,
                       int sh, int sw, int dh, int dw, int groups, int act,
                       pet_hip_stream_t stream);

/* pet_hip_conv2d_f32 for callers that cannot allocate device memory or have it
 * allocated on their behalf (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc). It has no counterpart in the reference. Same
 * arguments and results as pet_hip_conv2d_f32 in its run-to-run reproducible form
 * (partial sums of a split K loop added in a fixed order); the partial tiles live in
 * a static 8 MiB device array inside the library instead of the scratch that
 * pet_hip_init allocates, and the call itself allocates and frees nothing. A shape
 * whose split needs more than 8 MiB of partial tiles or more than 4096 output tiles
 * returns PET_HIP_ERR_UNSUPPORTED with the sizes in pet_hip_last_error(). All calls on
 * one GPU share that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race. */
PET_HIP_API int pet_hip_conv2d_static_f32(const float *x, const float *w, const float *bias,
                                          float *y, int n, int c, int h, int wd, int f, int r,
                                          int s, int ph, int pw, int sh, int sw, int dh, int dw,
                                          int groups, int act, pet_hip_stream_t stream);

/* Conv3d, NCTHW x [n,c,t,h,w], weight [f, c/groups, kt, r, s]. The reference
 * snapshot has no 3-D convolution (Operator::OpType, include/operator.h:19-51);
 * this is ConvOp::compute with one more spatial axis, needed by the ResNet3D-18
 * programs of pet-ae/run_policy_3d.sh:13-33. */
PET_HIP_API int pet_hip_conv3d_f32(const float *x, const float *w, const float *bias, float *y,
                       int n, int c, int t, int h, int wd, int f, int kt, int r, int s,
                       int pt, int ph, int pw, int st, int sh, int sw, int dt, int dh,
                       int dw, int groups, int act, pet_hip_stream_t stream);

/* The three contractions with a residual operand: y = act(op(x, w) + bias +
 * residual), residual laid out like y and not overlapping it. This is the z
 * operand of cudnnConvolutionBiasActivationForward, which the reference passes
 * with weight 0 (src/Graph/operator.cc:477-480, src/Graph/code_engine.cc:955-977);
 * a graph runtime uses it to run "convolution, then Add with another tensor,
 * then ReLU" (a ResNet block's tail) or "matmul, then Add" (a transformer
 * block's residual) as one operator. All other arguments as in the entry points
 * without _res; for the 3-D form w_is_packed says that w came from
 * pet_hip_conv3d_pack_filters. */
PET_HIP_API int pet_hip_conv2d_res_f32(const float *x, const float *w, const float *bias,
                           const float *residual, float *y, int n, int c, int h, int wd, int f,
                           int r, int s, int ph, int pw, int sh, int sw, int dh, int dw,
                           int groups, int act, pet_hip_stream_t stream);
PET_HIP_API int pet_hip_conv3d_res_f32(const float *x, const float *w, int w_is_packed,
                           const float *bias, const float *residual, float *y, int n, int c,
                           int t, int h, int wd, int f, int kt, int r, int s, int pt, int ph,
                           int pw, int st, int sh, int sw, int dt, int dh, int dw, int groups,
                           int act, pet_hip_stream_t stream);
PET_HIP_API int pet_hip_bmm_res_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                        const float *B, float *C, const float *bias, const float *residual,
                        int act, pet_hip_stream_t stream);

/* Matmul with every optional operand; flags: PET_HIP_CALL_Y_INITIALISED and
 * PET_HIP_CONV_ALGO(a) (the same K-sharing algorithms; transposed operands and k not a
 * multiple of 32 run on the general kernel, which has one). */
PET_HIP_API int pet_hip_bmm_ex_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                       const float *B, float *C, const float *bias, const float *residual, int act,
                       unsigned flags, pet_hip_stream_t stream);
PET_HIP_API int pet_hip_bmm_accumulates(int transA, int transB, int b, int m, int n, int k, int *yes);

/* Constant 3-D filters, reordered once: [f][c/groups][kt][r][s] -> kt-major
 * [kt][f][c/groups][r][s] (same element count), so that each kt slice is a 2-D
 * filter bank the convolution kernel reads with 16-byte loads. This is a
 * single-input operator on a Weight tensor, i.e. what the reference's emitted
 * program runs once before its timed loop ("Preprocess operators for weights",
 * src/Graph/code_engine.cc:187-193). Returns PET_HIP_ERR_UNSUPPORTED, writing
 * nothing, for shapes that would not profit (kt == 1, or filters other than
 * 3x3 with c/groups % 8 == 0 and 1x1 with c/groups % 32 == 0): keep calling
 * pet_hip_conv3d_f32 for those. */
PET_HIP_API int pet_hip_conv3d_pack_filters(const float *w, float *packed, int f, int cpg, int kt,
                                int r, int s, pet_hip_stream_t stream);

/* pet_hip_conv3d_f32 on filters reordered by pet_hip_conv3d_pack_filters; same
 * arguments and results. PET_HIP_ERR_UNSUPPORTED for the shapes that function
 * rejects. */
PET_HIP_API int pet_hip_conv3d_packed_f32(const float *x, const float *packed, const float *bias,
                              float *y, int n, int c, int t, int h, int wd, int f, int kt, int r,
                              int s, int pt, int ph, int pw, int st, int sh, int sw, int dt,
                              int dh, int dw, int groups, int act, pet_hip_stream_t stream);

/* The same contractions with every optional operand and the flags above, for graph
 * runtimes (the host layer's CodeEngine plans them): a split or stream-K launch
 * normally runs as "initialise y, accumulate, activate"; with the initialisations of a
 * whole graph batched into one pet_hip_bias_fill_batch launch at its start, and ReLU
 * left to the convolutions that read y, it is one launch. */
PET_HIP_API int pet_hip_conv2d_ex_f32(const float *x, const float *w, const float *bias,
                          const float *residual, float *y, int n, int c, int h, int wd, int f,
                          int r, int s, int ph, int pw, int sh, int sw, int dh, int dw, int groups,
                          int act, unsigned flags, pet_hip_stream_t stream);
PET_HIP_API int pet_hip_conv3d_ex_f32(const float *x, const float *w, int w_is_packed, const float *bias,
                          const float *residual, float *y, int n, int c, int t, int h, int wd,
                          int f, int kt, int r, int s, int pt, int ph, int pw, int st, int sh,
                          int sw, int dt, int dh, int dw, int groups, int act, unsigned flags,
                          pet_hip_stream_t stream);
/* A 2-D convolution operand addressed through strides, all counted in floats: element
 * (n, c, h, w) sits at n0 * n_stride[0] + n1 * n_stride[1] + n2 * n_stride[2] + c * c_stride +
 * h * h_stride + w * w_stride, where the batch index is taken apart innermost first:
 * n = (n2 * n_extent[1] + n1) * n_extent[0] + n0 (extent 1 for a factor that is not needed;
 * the strides of factors of extent 1 are not looked at). The strides must visit every float
 * of a dense buffer of n * c * h * w floats exactly once. */
typedef struct pet_hip_conv_view {
    long long c_stride, h_stride, w_stride;
    int n_extent[2];
    long long n_stride[3];
} pet_hip_conv_view;

/* pet_hip_conv2d_ex_f32 with x and / or y (and the residual, which is laid out like y) behind
 * such strides; NULL for an operand in its usual layout. This is how a layout operator next
 * to a convolution costs no launch: PET's space-to-batch Transpose in front of a convolution
 * (src/Mutant/generator.cc, the dilated-to-dense mutation; TransposeOp::compute,
 * src/Graph/operator.cc:2227-2245) is an x_view over the untransposed tensor, the
 * batch-to-space Transpose behind one a y_view over its output. No counterpart upstream, where
 * each Transpose is a kernel of its own. The sums are the ones pet_hip_conv2d_ex_f32 computes
 * on the transposed copy, in the same order. PET_HIP_ERR_UNSUPPORTED, nothing written, for
 * shapes outside pet_hip_conv2d_view_supported. */
PET_HIP_API int pet_hip_conv2d_view_f32(const float *x, const pet_hip_conv_view *x_view, const float *w,
                            const float *bias, const float *residual, float *y,
                            const pet_hip_conv_view *y_view, int n, int c, int h, int wd, int f,
                            int r, int s, int ph, int pw, int sh, int sw, int dh, int dw,
                            int groups, int act, unsigned flags, pet_hip_stream_t stream);
/* *yes = 1 when pet_hip_conv2d_view_f32 takes this shape (n, c, h, wd: the logical input):
 * 3x3 filters over a multiple of 8 channels per group or 1x1 filters over a multiple of 32,
 * operands below 2 GiB. */
PET_HIP_API int pet_hip_conv2d_view_supported(int n, int c, int h, int wd, int f, int r, int s, int ph,
                                  int pw, int sh, int sw, int dh, int dw, int groups, int *yes);
/* *yes = 1 when a launch of this shape accumulates into y with atomics (and so starts
 * by writing bias into all of y, unless told that y is initialised). Depends on the
 * shape and on PET_HIP_DETERMINISTIC only. */
PET_HIP_API int pet_hip_conv2d_accumulates(int n, int c, int h, int wd, int f, int r, int s, int ph,
                               int pw, int sh, int sw, int dh, int dw, int groups, int *yes);
PET_HIP_API int pet_hip_conv3d_accumulates(int n, int c, int t, int h, int wd, int f, int kt, int r,
                               int s, int pt, int ph, int pw, int st, int sh, int sw, int dt,
                               int dh, int dw, int groups, int w_is_packed, int *yes);
/* y[o][c][i] = bias[c] for `count` outputs in one launch (a convolution's output is
 * [n][f][pixels], a matmul's [b*m][n][1]). */
PET_HIP_API int pet_hip_bias_fill_batch(const pet_hip_fill *fills, int count, pet_hip_stream_t stream);

/* Batched row-major matmul C[b,m,n] = A'[b,m,k] * B'[b,k,n]; transA: A stored
 * [b,k,m]; transB: B stored [b,n,k]. bias (may be NULL) is [n], added per
 * output column. Semantics: MatmulOp::compute, src/Graph/operator.cc:620-654;
 * replaces cublasGemmStridedBatchedEx / cublasGemmEx
 * (src/Graph/operator.cc:777-780, 807-810; src/Graph/code_engine.cc:1103-1169). */
PET_HIP_API int pet_hip_bmm_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                    const float *B, float *C, const float *bias, int act,
                    pet_hip_stream_t stream);

/* Transposed convolution: x NHWF [n,h,w,f], weight RSFC [r,s,f,c], y NHWC [n,oh,ow,c],
 * oh = pet_hip_conv_trans_out_dim(h, r, ph, sh, dh, oph). Semantics: ConvTransOp::compute,
 * src/Graph/operator.cc:932-983 (flipped taps, input row (hh + rr*dh - (r-ph-1)) / sh where
 * exact, taps rr > r - (h + 2ph - r) % sh left out) over the output's own rows and columns,
 * i.e. the values of src/Test/convtrans_test_1.cc:62-77, 120-135; shape rule
 * ConvTransOp::computeShape, :1055-1072. bias (may be NULL) is [c]. Replaces
 * cudnnConvolutionBackwardData (src/Graph/operator.cc:1113-1287, src/Graph/code_engine.cc:
 * 979-1101). */
PET_HIP_API int pet_hip_conv_trans_out_dim(int i, int k, int p, int s, int d, int op);
PET_HIP_API int pet_hip_conv_trans_f32(const float *x, const float *w, const float *bias, float *y,
                           int n, int h, int wd, int f, int r, int s, int c, int ph, int pw,
                           int sh, int sw, int dh, int dw, int oph, int opw, int act,
                           pet_hip_stream_t stream);

/* Band products of sliding-window attention. G2BMM: A, B [bs,m,k] -> C [bs,m,2w+1],
 * C[b,i,j] = sum_k A[b,i,k] * B[b, i + d*(j-w), k]; GBMML: A [bs,m,2w+1], B [bs,m,n] ->
 * C [bs,m,n], C[b,i,x] = sum_j A[b,i,j] * B[b, i + d*j - d*w, x]; rows of B outside [0, m)
 * read as zero. Definitions: Sg2bmmPattern::getExpr / LongformerGBMMPattern::getExpr,
 * src/nnet/iterator_table.cc:596-630 (G2BMMOp / GBMMLOp have no CPU compute,
 * src/Graph/operator.cc:1355-1364, 1498-1507). Replace _sg2bmm / _sgbmml, the generated
 * kernels of include/custom_ops.cuh:3538-3559, 5778-5800 (src/Graph/operator.cc:1442-1463). */
PET_HIP_API int pet_hip_g2bmm_f32(const float *A, const float *B, float *C, int bs, int m, int k,
                      int width, int dilation, pet_hip_stream_t stream);
PET_HIP_API int pet_hip_gbmml_f32(const float *A, const float *B, float *C, int bs, int m, int width,
                      int n, int dilation, pet_hip_stream_t stream);

/* Multi-head attention core in one launch: for each batch entry and head h,
 * out[:, h*dh:(h+1)*dh] = softmax(scale * Q_h K_h^T) V_h, with Q, K, V [seq, heads*dh]
 * matrices whose rows are ldq / ldk / ldv floats apart (so the three slabs of a merged
 * projection, or three separate projections, are read in place) and out [seq, heads*dh]
 * with row stride ldo; the stride_* are the distances between batch entries. scale is
 * multiplied by *scale_dev when that is not NULL (a one-element tensor in the graph).
 * It stands for the operator sequence Transpose (head split) x 3, Matmul(transB), Mul,
 * Softmax, Matmul, Transpose (head merge), Reshape, i.e. MatmulOp::compute
 * (src/Graph/operator.cc:620-654) twice around a row softmax; the reference emits those
 * as cuBLAS calls and an inline softmax (src/Graph/code_engine.cc:1103-1169, 1707-1731).
 * seq <= 512, dh in {32, 64, 96, 128}, Q and K rows 16-byte aligned; PET_HIP_ERR_UNSUPPORTED
 * otherwise (callers then run the operators one by one). */
PET_HIP_API int pet_hip_attention_f32(const float *q, const float *k, const float *v, float *out,
                          int batch, int heads, int seq, int dh, int ldq, int ldk, int ldv,
                          int ldo, long long stride_q, long long stride_k, long long stride_v,
                          long long stride_o, float scale, const float *scale_dev,
                          pet_hip_stream_t stream);

/* ---- memory-bound operators given as an index expression ------------------------------
 * MemBoundOp::compute (src/Graph/operator.cc:3601-3644) evaluates, for every output
 * position, an expression tree (include/nnet/expr.h) with nnet::Interpreter
 * (src/nnet/Visitor/Interpreter.cc:31-131); the emitted program runs a TVM kernel printed
 * from the same tree (src/Graph/code_engine.cc:1752-1798). Here the tree is flattened into a
 * program of 32-bit integers for a small stack machine with an integer stack (index
 * arithmetic), a value stack (fp32) and iterator slots:
 *
 *   header  PET_HIP_EXPR_MAGIC, ntensors, {rank, extents...} per tensor, out_rank, extents...
 *   body    instructions, below; execution starts with the output position (outermost dim
 *           first) on the integer stack and ends at END with one value, the output element.
 *
 * ICONST v | IVAR slot: push. IADD ISUB IMUL IDIV IMOD: pop b, a, push a op b (C integer
 * division). LOAD t: pop rank(t) indices (last dim on top), push the element, 0 outside the
 * tensor (TensorNode::getData, src/nnet/expr.cc:62-72). I2F: move the integer top to the value
 * stack. FADD FSUB FMUL FDIV FMOD: value arithmetic (FDIV truncates, the reference's values
 * being integers). FRELU FTANH: in place. RANGE nloop skip {slot left right pad}*: pop nloop
 * positions into the slots; when one lies outside [left, right) push 0 and continue at word
 * `skip` (a range read in its padding, Interpreter.cc:63-72). SUM nsum {slot lo hi}*: set the
 * slots to lo, push an accumulator 0. SUMEND nsum body {slot lo hi}*: pop v, add it to the
 * accumulator below, step the iterators (last fastest); back to word `body` until they wrap,
 * then the accumulator is the value of the sum. Limits: 8 tensors, 32 slots, stacks 16 deep. */
#define PET_HIP_EXPR_MAGIC 0x50455401
typedef enum pet_hip_expr_op {
    PET_HIP_EXPR_END = 0,
    PET_HIP_EXPR_ICONST,
    PET_HIP_EXPR_IVAR,
    PET_HIP_EXPR_IADD,
    PET_HIP_EXPR_ISUB,
    PET_HIP_EXPR_IMUL,
    PET_HIP_EXPR_IDIV,
    PET_HIP_EXPR_IMOD,
    PET_HIP_EXPR_LOAD,
    PET_HIP_EXPR_I2F,
    PET_HIP_EXPR_FADD,
    PET_HIP_EXPR_FSUB,
    PET_HIP_EXPR_FMUL,
    PET_HIP_EXPR_FDIV,
    PET_HIP_EXPR_FMOD,
    PET_HIP_EXPR_FRELU,
    PET_HIP_EXPR_FTANH,
    PET_HIP_EXPR_RANGE,
    PET_HIP_EXPR_SUM,
    PET_HIP_EXPR_SUMEND
} pet_hip_expr_op;
/* Checks a program and keeps a copy of it in device memory (release it with pet_hip_free). */
PET_HIP_API int pet_hip_expr_program_create(const int *code, int ncode, int **device_code);
/* out[position] = program(position) for every position of the output shape in the header;
 * inputs[t] is tensor t of the header, contiguous. device_code comes from
 * pet_hip_expr_program_create for the same code. */
PET_HIP_API int pet_hip_expr_f32(const int *code, int ncode, const int *device_code,
                     const float *const *inputs, int ninputs, float *out,
                     pet_hip_stream_t stream);

/* ---- layout operators (bit-exact copies) ---------------------------------*/

/* TransposeOp::compute after the split has been resolved to flat dims,
 * src/Graph/operator.cc:2172-2210: view x as `flat_dims` (nflat <= 8), output
 * is that view permuted by `perm` (output dim j is flat dim perm[j]). Replaces
 * the TVM gather kernel and kernel_transpose_3d (src/Graph/code_engine.cc:27-84,
 * 499-530). */
PET_HIP_API int pet_hip_transpose(const float *x, float *y, const int *flat_dims, const int *perm,
                      int nflat, pet_hip_stream_t stream);

/* A TransSplit / TransReorder / TransFuse chain with its boundary-correction
 * parameters, src/Transpose/transpose.cc:22-42 (split: extr, copys), 136-150
 * (reorder), 70-106 (fuse: pad, dels); what TransposeEngine::getLambda (:192-220)
 * hands to TVM. ops holds nops records of 6 ints {kind, a, b, c, d, 0}:
 *   kind 0 split  : a=index, b=in_dim, c=extr, d=copys
 *   kind 1 reorder: permutation read from `perms` (rank-at-that-point ints)
 *   kind 2 fuse   : a=index, b=pad, c=dels
 * out_dims (PET_HIP_MAX_RANK ints) receives the result shape, *out_rank its
 * rank. With y == NULL only the shape is computed. Positions that map outside
 * the input, and the pad rows of a fuse, are written as 0. */
PET_HIP_API int pet_hip_trans_chain(const float *x, float *y, const int *in_dims, int rank,
                        const int *ops, int nops, const int *perms, int *out_dims,
                        int *out_rank, pet_hip_stream_t stream);

/* SplitOp::computeV, src/Graph/operator.cc:1978-2020: ys[i] receives the slab
 * of extent out_sizes[i] along `dim` (sum must equal in_dims[dim]). Replaces
 * the pointer aliasing / TVM kernels of src/Graph/code_engine.cc:133-144,
 * 1505-1545. */
PET_HIP_API int pet_hip_split(const float *x, float *const *ys, int k, const int *in_dims, int rank,
                  int dim, const int *out_sizes, pet_hip_stream_t stream);

/* ConcatOp::compute, src/Graph/operator.cc:1813-1850 (inputs may repeat).
 * Replaces src/Graph/code_engine.cc:145-154, 1551-1615. */
PET_HIP_API int pet_hip_concat(const float *const *xs, int k, float *y, const int *out_dims, int rank,
                   int dim, const int *in_sizes, pet_hip_stream_t stream);

/* PadOp::compute, src/Graph/operator.cc:1640-1662 (cudnnTransformTensorEx at
 * src/Graph/code_engine.cc:1171-1216). */
PET_HIP_API int pet_hip_pad(const float *x, float *y, const int *in_dims, const int *begin,
                const int *end, int rank, pet_hip_stream_t stream);

/* SliceOp::compute, src/Graph/operator.cc:1741-1756
 * (src/Graph/code_engine.cc:1465-1499). */
PET_HIP_API int pet_hip_slice(const float *x, float *y, const int *in_dims, const int *begin,
                  const int *end, int rank, pet_hip_stream_t stream);

/* ExtendOp::compute, src/Graph/operator.cc:2577-2597: the block from `dim`
 * inwards repeated num+1 times (src/Graph/code_engine.cc:1621-1675). */
PET_HIP_API int pet_hip_extend(const float *x, float *y, const int *in_dims, int rank, int dim,
                   int num, pet_hip_stream_t stream);

/* ---- element-wise ---------------------------------------------------------*/

/* k-ary Add / Mul, binary Sub / Div with flat-modulo broadcast in[i % sizes[j]]
 * (src/Graph/operator.cc:2983-3002, 3074-3090, 3157-3176); replaces
 * cublasSaxpy / cudnnOpTensor (src/Graph/code_engine.cc:1335-1348, 1377-1422).
 * k <= 8. y may alias ins[j] only when sizes[j] == n. */
PET_HIP_API int pet_hip_eltwise(int op, const float *const *ins, const size_t *sizes, int k, float *y,
                    size_t n, pet_hip_stream_t stream);

/* PowOp::compute, src/Graph/operator.cc:3330-3343 with powVType
 * (include/common.h:157-162): y = 1 * x * x ... (`pow` factors, each product rounded
 * to fp32; pow <= 0 gives 1). pow <= 1024. x == y is allowed. */
PET_HIP_API int pet_hip_pow(const float *x, float *y, size_t n, int pow, pet_hip_stream_t stream);

/* BatchNormOp::compute, src/Graph/operator.cc:2660-2681, on an [outer, ch, inner]
 * view (channel = dim 1 of the tensor): y = (x - mean[ch]) * scale[ch] /
 * sqrt(var[ch] + eps) + bias[ch]. The reference emits nothing for it on the GPU
 * (src/Graph/code_engine.cc:1848-1850). x == y is allowed. */
PET_HIP_API int pet_hip_batchnorm(const float *x, const float *scale, const float *bias,
                      const float *mean, const float *var, float *y, size_t outer, size_t ch,
                      size_t inner, float eps, pet_hip_stream_t stream);

/* GatherOp: out[j..., p..., q...] = x[p..., indices[j...], q...], the index dims
 * leading the output (GatherOp::computeShape, src/Graph/operator.cc:3420-3428, and
 * the lambda of CodeEngine::genGatherCompute, src/Graph/code_engine.cc:1465-1498,
 * which this replaces). pre / post: products of the dims of x before / after the
 * axis, dim: the axis extent, nidx: number of indices. indices: int32, or fp32
 * values holding integers when index_is_float != 0. Negative indices count from the
 * end; indices outside the axis give zeros. The reference has no CPU compute for it
 * (src/Graph/operator.cc:3409-3412). */
PET_HIP_API int pet_hip_gather(const float *x, const void *indices, int index_is_float, float *y,
                   size_t pre, size_t dim, size_t post, size_t nidx, pet_hip_stream_t stream);

/* ReduceMeanOp: y[o, 0, i] = mean over d of x[o, d, i] (shape rule
 * ReduceMeanOp::computeShape, src/Graph/operator.cc:3454-3458; no CPU compute and no
 * GPU emitter upstream, :3443-3446). */
PET_HIP_API int pet_hip_reduce_mean(const float *x, float *y, size_t outer, size_t dim, size_t inner,
                        pet_hip_stream_t stream);

/* y = act(x); replaces cudnnActivationForward (src/Graph/code_engine.cc:1260-1274).
 * The reference has no CPU compute for it (include/operator.h:1968-1977). */
PET_HIP_API int pet_hip_activation(const float *x, float *y, size_t n, int act, pet_hip_stream_t stream);

/* y[o, ch, i] = act(x[o, ch, i] + bias[ch]) on an [outer, ch, inner] view;
 * replaces cudnnAddTensor + cudnnActivationForward
 * (src/Graph/code_engine.cc:917-924, 944-952). x == y is allowed. */
PET_HIP_API int pet_hip_bias_act(const float *x, const float *bias, float *y, size_t outer, size_t ch,
                     size_t inner, int act, pet_hip_stream_t stream);

/* ---- non-contraction network pieces without a reference CPU compute -------*/

/* Max (mode 0) / average (mode 1) pooling over NCHW with
 * out = (in + 2p - d (k-1) - 1) / s + 1. The average divides by the number of
 * window positions inside the image (CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING,
 * src/Graph/operator.cc:2933). Replaces cudnnPoolingForward
 * (src/Graph/operator.cc:2814-2827, 2937-2950; code_engine.cc:1315-1329). */
PET_HIP_API int pet_hip_pool2d(const float *x, float *y, int n, int c, int h, int w, int kh, int kw,
                   int ph, int pw, int sh, int sw, int dh, int dw, int mode,
                   pet_hip_stream_t stream);
/* The same with pet_hip_call_flags: PET_HIP_CALL_X_RELU pools max(x, 0) (the ReLU of the
 * convolution that produced x, left to this reader; cuDNN's fused activation has no such
 * hand-over, src/Graph/code_engine.cc:955-977 applies it in the producer). */
PET_HIP_API int pet_hip_pool2d_ex(const float *x, float *y, int n, int c, int h, int w, int kh, int kw,
                      int ph, int pw, int sh, int sw, int dh, int dw, int mode, unsigned flags,
                      pet_hip_stream_t stream);

/* Row softmax over the last axis of a [rows, cols] view; replaces
 * online_softmax (src/Graph/code_engine.cc:424-486, 1707-1731). */
PET_HIP_API int pet_hip_softmax(const float *x, float *y, size_t rows, size_t cols,
                    pet_hip_stream_t stream);

/* LayerNorm over the last axis (gamma / beta may be NULL); absent upstream,
 * needed by the BERT-base-shaped encoder. */
PET_HIP_API int pet_hip_layernorm(const float *x, const float *gamma, const float *beta, float *y,
                      size_t rows, size_t cols, float eps, pet_hip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PET_HIP_H */
