/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU oracle for the PET operator path: a plain-C restatement of the reference's
 * Operator::compute bodies (src/Graph/operator.cc) and of the transpose index
 * algebra (src/Transpose/transpose.cc). Nothing in the shipped library links or
 * loads this file; only the test-suite, the smoke check and the benchmark's CPU
 * baseline leg do.
 *
 * Two tiers are generated from pet_oracle_ops.inc:
 *   *_u32 : storage and accumulation in wrapping uint32, exactly the reference's
 *           VType (include/common.h:137);
 *   *_f32 : fp32 storage with fp64 accumulation for contractions, the tier the
 *           fp32 GPU kernels are compared against.
 *
 * Pinning status (what checks each function besides this restatement):
 *   conv2d, conv2d_point : torch.nn.functional.conv2d (CPU) incl. stride,
 *       dilation, groups; full == point-wise identity (src/Test/conv_test_3.cc);
 *       hand-computed 1-D cases.
 *   conv3d : kt=1 reduction to conv2d; torch.nn.functional.conv3d (CPU). The
 *       reference has no Conv3d, so reference parity is unpinned by construction.
 *   matmul : numpy.matmul with explicit transposes; hand values of
 *       src/Test/batch_gemm_test.cc:45-50.
 *   transpose : numpy reshape/transpose/reshape closed forms given by
 *       src/Test/transpose_test_2.py:4-31 and dat/transpose_test/transpose_ops.op.
 *   split_one, concat_one, pad, slice, extend : numpy split / concatenate / pad /
 *       slicing / tile.
 *   eltwise : numpy with explicit flat-modulo broadcast on hand-built cases.
 *   pow : Python integers modulo 2^32 (u32 tier) and numpy integer powers of small
 *       integers, exact in fp32 (f32 tier); pow 0 and 1 by definition.
 *   div : numpy true division. The reference's DivOp::compute body subtracts
 *       (src/Graph/operator.cc:3259) and nothing upstream runs Div on a GPU, so
 *       division itself is parity unpinned by the reference.
 *   gather, reduce_mean : numpy.take + moveaxis / numpy.mean(keepdims). The reference
 *       holds shape rules only (src/Graph/operator.cc:3409-3458): parity unpinned by it.
 *   batchnorm : torch.nn.functional.batch_norm (CPU, inference mode) and the
 *       identity statistics (mean 0, var 1 - eps, scale 1, bias 0 -> y = x).
 *   trans_chain : numpy constructions of halo split / drop fuse / pad fuse /
 *       extr split on iota inputs, and conv equivalence (split+conv+fuse == conv).
 *   relu/sigmoid/tanh/gelu, bias_act, maxpool, avgpool, softmax, layernorm :
 *       parity unpinned by the reference (ActivationOp / MaxPoolOp / AvgPoolOp /
 *       SoftmaxOp::compute are assert(false), include/operator.h:1968-1977,
 *       src/Graph/operator.cc:2746-2750, 2871-2875, 3409-3412; GELU and LayerNorm
 *       do not exist there); pinned by closed forms and torch CPU routines.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define PET_ORACLE_EXPORT __attribute__((visibility("default")))

#define T uint32_t
#define ACC uint32_t
#define FN(name) PET_ORACLE_EXPORT oracle_##name##_u32
#include "pet_oracle_ops.inc"
#undef T
#undef ACC
#undef FN

#define T float
#define ACC double
#define FN(name) PET_ORACLE_EXPORT oracle_##name##_f32
#include "pet_oracle_ops.inc"
#undef T
#undef ACC
#undef FN

/* ConvOp::computeShape with explicit padding, src/Graph/operator.cc:219-221:
 * o = (i - (k - s) * d + 2 p) / s. Equals the textbook floor formula unless
 * d > 1 and s > 1. */
PET_ORACLE_EXPORT int oracle_conv_out_dim(int i, int k, int p, int s, int d) {
    return (i - (k - s) * d + p * 2) / s;
}

/* ConvOp::computeShape in Same mode, src/Graph/operator.cc:222-226. */
PET_ORACLE_EXPORT void oracle_conv_same(int i, int k, int s, int d, int *o,
                                        int *p) {
    *o = i / s;
    *p = (i - *o * s + (k - s) * d) / 2;
}

/* Tensor::fastrand, include/tensor.h:371-374, single stream. The reference
 * draws data[i] = fastrand(seed_of_thread) % 10000 with one seed per OpenMP
 * thread (tensor.h:180-182), so its tensors depend on the thread count; this
 * is the one-thread stream, seed 0 as initFastrand sets for thread 0. */
PET_ORACLE_EXPORT void oracle_fastrand_fill(uint32_t *dst, size_t n, int seed,
                                            uint32_t mod) {
    int g = seed;
    for (size_t i = 0; i < n; ++i) {
        g = (int)(214013u * (uint32_t)g + 2531011u);
        uint32_t v = (uint32_t)((g >> 16) & 0x7FFF);
        dst[i] = mod ? v % mod : v;
    }
}

PET_ORACLE_EXPORT int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- fp32-only element-wise pieces (no reference CPU compute exists) ---- */

static inline float act_apply(int act, float v) {
    switch (act) {
    case 1:
        return v > 0.f ? v : 0.f;
    case 2:
        return (float)(1.0 / (1.0 + exp(-(double)v)));
    case 3:
        return (float)tanh((double)v);
    case 4: /* exact GELU: x * Phi(x) */
        return (float)(0.5 * (double)v * (1.0 + erf((double)v * M_SQRT1_2)));
    default:
        return v;
    }
}

/* ActType order of include/operator.h:95-100 (None, Relu, Sigmoid, Tanh), plus
 * 4 = GELU which the reference lacks. */
PET_ORACLE_EXPORT void oracle_activation_f32(const float *x, float *y, size_t n,
                                             int act) {
#pragma omp parallel for
    for (size_t i = 0; i < n; ++i)
        y[i] = act_apply(act, x[i]);
}

/* DivOp with the flat-modulo broadcast of the other binary operators
 * (shape rule src/Graph/operator.cc:3306-3313). The reference's compute body
 * at :3259 subtracts; this is division. */
PET_ORACLE_EXPORT void oracle_div_f32(const float *a, size_t na, const float *b, size_t nb,
                                      float *y, size_t n) {
#pragma omp parallel for
    for (size_t i = 0; i < n; ++i)
        y[i] = a[i % na] / b[i % nb];
}

/* BatchNormOp::compute, src/Graph/operator.cc:2660-2681: channel = dim 1,
 * factor[c] = scale[c] / sqrt(var[c] + eps) in double, y = (x - mean[c]) *
 * factor[c] + bias[c]. */
PET_ORACLE_EXPORT void oracle_batchnorm_f32(const float *x, const float *scale,
                                            const float *bias, const float *mean,
                                            const float *var, float *y, size_t outer,
                                            size_t ch, size_t inner, float eps) {
#pragma omp parallel for
    for (size_t i = 0; i < outer * ch * inner; ++i) {
        size_t c = (i / inner) % ch;
        double factor = (double)scale[c] / sqrt((double)var[c] + (double)eps);
        y[i] = (float)(((double)x[i] - (double)mean[c]) * factor + (double)bias[c]);
    }
}

/* GatherOp as the reference's shape rule and GPU lambda define it
 * (src/Graph/operator.cc:3420-3428, src/Graph/code_engine.cc:1465-1498):
 * out[j, p, q] = x[p, idx[j], q]; negative indices count from the end, indices
 * outside the axis give 0. */
PET_ORACLE_EXPORT void oracle_gather_f32(const float *x, const int *idx, float *y, size_t pre,
                                         size_t dim, size_t post, size_t nidx) {
    for (size_t j = 0; j < nidx; ++j) {
        long long id = idx[j];
        if (id < 0)
            id += (long long)dim;
        for (size_t p = 0; p < pre; ++p)
            for (size_t q = 0; q < post; ++q)
                y[(j * pre + p) * post + q] =
                    (id >= 0 && id < (long long)dim) ? x[(p * dim + (size_t)id) * post + q] : 0.f;
    }
}

/* ReduceMeanOp (shape rule src/Graph/operator.cc:3454-3458): mean over the axis in
 * double. */
PET_ORACLE_EXPORT void oracle_reduce_mean_f32(const float *x, float *y, size_t outer, size_t dim,
                                              size_t inner) {
    for (size_t o = 0; o < outer; ++o)
        for (size_t i = 0; i < inner; ++i) {
            double s = 0.0;
            for (size_t d = 0; d < dim; ++d)
                s += (double)x[(o * dim + d) * inner + i];
            y[o * inner + i] = (float)(s / (double)dim);
        }
}

/* y[o, ch, inner] = act(x + bias[ch]): the epilogue the GPU path fuses
 * (cudnnConvolutionBiasActivationForward at src/Graph/operator.cc:478-481 is
 * what the reference times; its CPU compute ignores bias and act). */
PET_ORACLE_EXPORT void oracle_bias_act_f32(const float *x, const float *bias,
                                           float *y, size_t outer, size_t ch,
                                           size_t inner, int act) {
#pragma omp parallel for
    for (size_t i = 0; i < outer * ch * inner; ++i) {
        size_t c = (i / inner) % ch;
        float v = x[i] + (bias ? bias[c] : 0.f);
        y[i] = act_apply(act, v);
    }
}

/* Max / average pooling over NCHW, cudnnPoolingForward semantics as used at
 * src/Graph/operator.cc:2814-2827, 2937-2950: out = (in + 2p - d*(k-1) - 1)/s + 1,
 * the average divides by the number of window positions inside the image
 * (CUDNN_POOLING_AVERAGE_COUNT_EXCLUDE_PADDING, src/Graph/operator.cc:2933,
 * src/Graph/code_engine.cc:1303). mode 0 = max, 1 = avg. */
PET_ORACLE_EXPORT void oracle_pool2d_f32(const float *x, float *y, int n, int c,
                                         int h, int w, int kh, int kw, int ph,
                                         int pw, int sh, int sw, int dh, int dw,
                                         int oh, int ow, int mode) {
#pragma omp parallel for
    for (int nc = 0; nc < n * c; ++nc) {
        const float *xp = x + (size_t)nc * h * w;
        float *yp = y + (size_t)nc * oh * ow;
        for (int i = 0; i < oh; ++i)
            for (int j = 0; j < ow; ++j) {
                double acc = mode == 0 ? -INFINITY : 0.0;
                int taps = 0;
                for (int r = 0; r < kh; ++r)
                    for (int s = 0; s < kw; ++s) {
                        int ih = i * sh + r * dh - ph, iw = j * sw + s * dw - pw;
                        if (ih < 0 || ih >= h || iw < 0 || iw >= w)
                            continue;
                        float v = xp[(size_t)ih * w + iw];
                        if (mode == 0)
                            acc = v > acc ? v : acc;
                        else
                            acc += v;
                        ++taps;
                    }
                yp[(size_t)i * ow + j] =
                    mode == 0 ? (float)acc : (float)(taps ? acc / (double)taps : 0.0);
            }
    }
}

/* Softmax over the last axis of a [rows, cols] view. */
PET_ORACLE_EXPORT void oracle_softmax_f32(const float *x, float *y, size_t rows,
                                          size_t cols) {
#pragma omp parallel for
    for (size_t r = 0; r < rows; ++r) {
        const float *xp = x + r * cols;
        float *yp = y + r * cols;
        double mx = -INFINITY, sum = 0;
        for (size_t j = 0; j < cols; ++j)
            mx = xp[j] > mx ? xp[j] : mx;
        for (size_t j = 0; j < cols; ++j)
            sum += exp((double)xp[j] - mx);
        for (size_t j = 0; j < cols; ++j)
            yp[j] = (float)(exp((double)xp[j] - mx) / sum);
    }
}

/* LayerNorm over the last axis: (x - mean) / sqrt(var + eps) * gamma + beta. */
PET_ORACLE_EXPORT void oracle_layernorm_f32(const float *x, const float *gamma,
                                            const float *beta, float *y,
                                            size_t rows, size_t cols,
                                            float eps) {
#pragma omp parallel for
    for (size_t r = 0; r < rows; ++r) {
        const float *xp = x + r * cols;
        float *yp = y + r * cols;
        double mean = 0, var = 0;
        for (size_t j = 0; j < cols; ++j)
            mean += xp[j];
        mean /= (double)cols;
        for (size_t j = 0; j < cols; ++j)
            var += ((double)xp[j] - mean) * ((double)xp[j] - mean);
        var /= (double)cols;
        double inv = 1.0 / sqrt(var + (double)eps);
        for (size_t j = 0; j < cols; ++j)
            yp[j] = (float)(((double)xp[j] - mean) * inv *
                                (gamma ? (double)gamma[j] : 1.0) +
                            (beta ? (double)beta[j] : 0.0));
    }
}
