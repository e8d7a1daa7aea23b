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
 *   conv_trans : the golden vectors of the reference's own tests
 *       (src/Test/convtrans_test_1.cc:62-77, 120-135, convtrans_test_2.cc:81-82, 144-145),
 *       reproduced exactly; torch.nn.functional.conv_transpose2d (CPU) on strided, padded
 *       and output-padded shapes; the tap skip of src/Graph/operator.cc:957-960 as torch's
 *       result on a kernel with the skipped rows zeroed. With dilation != 1 the reference's
 *       loop keeps the undilated offset r - ph - 1 (:961-962) and is an operator of its
 *       own: parity unpinned for dilated transposed convolution.
 *   g2bmm, gbmml : band products cut out of numpy's dense matmul, from the definitions
 *       of src/nnet/iterator_table.cc:596-630. The reference has no CPU compute for them
 *       (src/Graph/operator.cc:1424-1598 are shape rules): parity unpinned by it; on a GPU
 *       box the reference's nnet::Interpreter evaluates the same definitions.
 *   expr (MemBound programs) : numpy index maps, gathers and sums; on a GPU box the
 *       reference's nnet::Interpreter, compiled unchanged, on the same expressions.
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


/* ---- MemBoundOp: an index expression evaluated at every output position ------------
 * MemBoundOp::compute, src/Graph/operator.cc:3601-3644, runs nnet::Interpreter
 * (src/nnet/Visitor/Interpreter.cc) on the operator's expression tree for every output
 * position: Subscript of a tensor reads 0 outside the tensor (TensorNode::getData,
 * src/nnet/expr.cc:62-72), a RangeOp reached through a Subscript in its padding is 0
 * (Interpreter.cc:63-72), sum iterators run over [lo, hi) with the last one fastest
 * (:85-105), BinaryOp is C integer arithmetic on indices (:31-50). The tree arrives here
 * flattened into the integer program of include/pet_hip.h (same opcodes, copied below so
 * that this file needs nothing of the library); values are fp32, sums accumulate in fp64.
 * Pinned by numpy index maps (tests/test_oracle.py) and, where the reference tree is
 * present, by nnet::Interpreter itself on trees the reference builds
 * (tests/cpp/membound_driver.cc). Returns 0, or 1 for a malformed program. */
enum {
    EX_END, EX_ICONST, EX_IVAR, EX_IADD, EX_ISUB, EX_IMUL, EX_IDIV, EX_IMOD, EX_LOAD, EX_I2F,
    EX_FADD, EX_FSUB, EX_FMUL, EX_FDIV, EX_FMOD, EX_FRELU, EX_FTANH, EX_RANGE, EX_SUM, EX_SUMEND
};

PET_ORACLE_EXPORT int oracle_expr_f32(const int *code, int ncode, const float *const *in,
                                      float *out) {
    if (ncode < 4 || code[0] != 0x50455401)
        return 1;
    int at = 1, nt = code[at++];
    int nd[8], shape_at[8];
    if (nt < 0 || nt > 8)
        return 1;
    for (int t = 0; t < nt; ++t) {
        nd[t] = code[at++];
        shape_at[t] = at;
        at += nd[t];
    }
    const int out_nd = code[at++];
    const int *out_shape = code + at;
    at += out_nd;
    size_t total = 1;
    for (int d = 0; d < out_nd; ++d)
        total *= (size_t)out_shape[d];
    const int pc0 = at;
    int failed = 0;
#pragma omp parallel for
    for (size_t i = 0; i < total; ++i) {
        int istack[32], vars[32], isp = 0, fsp = 0;
        double fstack[32];
        size_t t = i;
        int pos[8];
        for (int j = out_nd - 1; j >= 0; --j) {
            pos[j] = (int)(t % (size_t)out_shape[j]);
            t /= (size_t)out_shape[j];
        }
        for (int j = 0; j < out_nd; ++j)
            istack[isp++] = pos[j];
        int pc = pc0;
        while (pc < ncode && code[pc] != EX_END) {
            const int op = code[pc];
            if (op == EX_ICONST) {
                istack[isp++] = code[pc + 1];
                pc += 2;
            } else if (op == EX_IVAR) {
                istack[isp++] = vars[code[pc + 1]];
                pc += 2;
            } else if (op >= EX_IADD && op <= EX_IMOD) {
                int b = istack[--isp], a = istack[--isp];
                istack[isp++] = op == EX_IADD   ? a + b
                                : op == EX_ISUB ? a - b
                                : op == EX_IMUL ? a * b
                                : op == EX_IDIV ? (b ? a / b : 0)
                                                : (b ? a % b : 0);
                pc += 1;
            } else if (op == EX_LOAD) {
                const int tn = code[pc + 1], n = nd[tn];
                const int *shape = code + shape_at[tn];
                isp -= n;
                size_t off = 0;
                int inside = 1;
                for (int d = 0; d < n; ++d) {
                    int idx = istack[isp + d];
                    if (idx < 0 || idx >= shape[d])
                        inside = 0;
                    off = off * (size_t)shape[d] + (size_t)(idx < 0 ? 0 : idx);
                }
                fstack[fsp++] = inside ? (double)in[tn][off] : 0.0;
                pc += 2;
            } else if (op == EX_I2F) {
                fstack[fsp++] = (double)istack[--isp];
                pc += 1;
            } else if (op >= EX_FADD && op <= EX_FMOD) {
                double b = fstack[--fsp], a = fstack[--fsp];
                fstack[fsp++] = op == EX_FADD   ? a + b
                                : op == EX_FSUB ? a - b
                                : op == EX_FMUL ? a * b
                                : op == EX_FDIV ? trunc(a / b)
                                                : fmod(a, b);
                pc += 1;
            } else if (op == EX_FRELU) {
                if (fstack[fsp - 1] < 0)
                    fstack[fsp - 1] = 0;
                pc += 1;
            } else if (op == EX_FTANH) {
                fstack[fsp - 1] = tanh(fstack[fsp - 1]);
                pc += 1;
            } else if (op == EX_RANGE) {
                const int n = code[pc + 1], skip = code[pc + 2];
                isp -= n;
                int inside = 1;
                for (int d = 0; d < n; ++d) {
                    const int *it = code + pc + 3 + 4 * d;
                    vars[it[0]] = istack[isp + d];
                    if (istack[isp + d] < it[1] || istack[isp + d] >= it[2])
                        inside = 0;
                }
                if (inside) {
                    pc += 3 + 4 * n;
                } else {
                    fstack[fsp++] = 0.0;
                    pc = skip;
                }
            } else if (op == EX_SUM) {
                const int n = code[pc + 1];
                for (int d = 0; d < n; ++d)
                    vars[code[pc + 2 + 3 * d]] = code[pc + 3 + 3 * d];
                fstack[fsp++] = 0.0;
                pc += 2 + 3 * n;
            } else if (op == EX_SUMEND) {
                const int n = code[pc + 1], body = code[pc + 2];
                double v = fstack[--fsp];
                fstack[fsp - 1] += v;
                int d = n - 1;
                for (; d >= 0; --d) {
                    const int *it = code + pc + 3 + 3 * d;
                    if (++vars[it[0]] < it[2])
                        break;
                    vars[it[0]] = it[1];
                }
                pc = d >= 0 ? body : pc + 3 + 3 * n;
            } else {
                failed = 1;
                break;
            }
        }
        out[i] = fsp > 0 ? (float)fstack[fsp - 1] : 0.f;
    }
    return failed;
}
