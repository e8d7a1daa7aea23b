// Element-wise operators, activation / bias epilogues and the small
// non-contraction network pieces (pooling, softmax, layernorm).
#include "common.h"

#include <algorithm>
#include <cstring>

using namespace pet;

namespace {

constexpr int kMaxEltIn = 8;

struct EltParams {
    const float *in[kMaxEltIn];
    unsigned size[kMaxEltIn]; // 0 = same size as the output (no modulo)
    unsigned mul[kMaxEltIn], shift[kMaxEltIn];
    int k, op;
    size_t n;
};

__device__ __forceinline__ unsigned mod_fast(unsigned i, unsigned d, unsigned mul, unsigned shift) {
    unsigned q = __umulhi(i, mul) >> shift;
    return i - q * d;
}

// VEC == 4: the host has checked n % 4 == 0, every broadcast size % 4 == 0 and
// 16-byte alignment, so four consecutive outputs read four consecutive inputs.
template <int VEC>
__global__ __launch_bounds__(256) void eltwise_kernel(EltParams p, float *__restrict__ y) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    const size_t step = (size_t)gridDim.x * 256 * VEC;
    for (; i < p.n; i += step) {
        float acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v)
            acc[v] = p.op == PET_HIP_MUL ? 1.f : 0.f;
#pragma unroll
        for (int j = 0; j < kMaxEltIn; ++j) {
            if (j < p.k) {
                size_t src = i;
                if (p.size[j] == 1)
                    src = 0;
                else if (p.size[j])
                    src = mod_fast((unsigned)i, p.size[j], p.mul[j], p.shift[j]);
                float val[VEC];
                if (VEC == 4 && p.size[j] != 1) {
                    float4 t = *reinterpret_cast<const float4 *>(p.in[j] + src);
                    val[0] = t.x;
                    val[1 % VEC] = t.y;
                    val[2 % VEC] = t.z;
                    val[3 % VEC] = t.w;
                } else {
#pragma unroll
                    for (int v = 0; v < VEC; ++v)
                        val[v] = p.in[j][p.size[j] == 1 ? 0 : src + v];
                }
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    if (p.op == PET_HIP_ADD)
                        acc[v] += val[v];
                    else if (p.op == PET_HIP_MUL)
                        acc[v] *= val[v];
                    else if (p.op == PET_HIP_SUB)
                        acc[v] = j == 0 ? val[v] : acc[v] - val[v];
                    else
                        acc[v] = j == 0 ? val[v] : acc[v] / val[v];
                }
            }
        }
        if (VEC == 4)
            *reinterpret_cast<float4 *>(y + i) = make_float4(acc[0], acc[1 % VEC], acc[2 % VEC],
                                                             acc[3 % VEC]);
        else
            y[i] = acc[0];
    }
}

template <int VEC>
__global__ __launch_bounds__(256) void activation_kernel(const float *__restrict__ x,
                                                         float *__restrict__ y, size_t n,
                                                         int act) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    const size_t step = (size_t)gridDim.x * 256 * VEC;
    for (; i < n; i += step) {
        if (VEC == 4) {
            float4 v = *reinterpret_cast<const float4 *>(x + i);
            v.x = apply_act(v.x, act);
            v.y = apply_act(v.y, act);
            v.z = apply_act(v.z, act);
            v.w = apply_act(v.w, act);
            *reinterpret_cast<float4 *>(y + i) = v;
        } else {
            y[i] = apply_act(x[i], act);
        }
    }
}

// y = x multiplied up `pow` times from 1, every product rounded to fp32 (the order
// of PowOp's CPU loop, so small integers and exact products agree bit for bit).
template <int VEC>
__global__ __launch_bounds__(256) void pow_kernel(const float *__restrict__ x,
                                                  float *__restrict__ y, size_t n, int pow) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    const size_t step = (size_t)gridDim.x * 256 * VEC;
    for (; i < n; i += step) {
        float v[VEC], r[VEC];
        if (VEC == 4) {
            float4 t = *reinterpret_cast<const float4 *>(x + i);
            v[0] = t.x;
            v[1 % VEC] = t.y;
            v[2 % VEC] = t.z;
            v[3 % VEC] = t.w;
        } else {
            v[0] = x[i];
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e)
            r[e] = 1.f;
        for (int j = 0; j < pow; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                r[e] *= v[e];
        if (VEC == 4)
            *reinterpret_cast<float4 *>(y + i) = make_float4(r[0], r[1 % VEC], r[2 % VEC],
                                                             r[3 % VEC]);
        else
            y[i] = r[0];
    }
}

// Inference batch normalisation over [outer, ch, inner]: one (outer, ch) row of
// `inner` elements per workgroup pass, so the channel's factor and shift are
// computed once per row and the row moves as 16-byte words when it can.
__global__ __launch_bounds__(256) void batchnorm_kernel(const float *__restrict__ x,
                                                        const float *__restrict__ scale,
                                                        const float *__restrict__ bias,
                                                        const float *__restrict__ mean,
                                                        const float *__restrict__ var,
                                                        float *__restrict__ y, size_t rows,
                                                        unsigned ch, size_t inner, float eps,
                                                        int vec) {
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const unsigned c = (unsigned)(row % ch);
        const float factor = scale[c] / sqrtf(var[c] + eps);
        const float shift = bias[c] - mean[c] * factor;
        const float *xr = x + row * inner;
        float *yr = y + row * inner;
        if (vec) {
            for (size_t i = threadIdx.x * 4; i < inner; i += 1024) {
                float4 v = *reinterpret_cast<const float4 *>(xr + i);
                v.x = v.x * factor + shift;
                v.y = v.y * factor + shift;
                v.z = v.z * factor + shift;
                v.w = v.w * factor + shift;
                *reinterpret_cast<float4 *>(yr + i) = v;
            }
        } else {
            for (size_t i = threadIdx.x; i < inner; i += 256)
                yr[i] = xr[i] * factor + shift;
        }
    }
}

// out[j, p, q] = x[p, idx[j], q]: the index dims lead the output, as in the
// reference's shape rule. Negative indices count from the end; an index outside
// the axis gives zeros.
template <bool FIDX>
__global__ __launch_bounds__(256) void gather_kernel(const float *__restrict__ x,
                                                     const void *__restrict__ indices,
                                                     float *__restrict__ y, size_t total,
                                                     size_t pre, long long dim, size_t post) {
    size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t step = (size_t)gridDim.x * 256;
    const size_t slab = pre * post;
    for (; o < total; o += step) {
        const size_t j = o / slab, r = o - j * slab;
        const size_t pi = r / post, q = r - pi * post;
        long long id = FIDX ? (long long)rintf(static_cast<const float *>(indices)[j])
                            : (long long)static_cast<const int *>(indices)[j];
        if (id < 0)
            id += dim;
        y[o] = (id >= 0 && id < dim) ? x[(pi * (size_t)dim + (size_t)id) * post + q] : 0.f;
    }
}

// y[o, i] = mean over d of x[o, d, i]. A thread owns one output and walks d
// (neighbouring threads read neighbouring i); with inner == 1 a wave owns one row
// and sums it across lanes.
__global__ __launch_bounds__(256) void reduce_mean_kernel(const float *__restrict__ x,
                                                          float *__restrict__ y, size_t outer,
                                                          size_t dim, size_t inner) {
    if (inner == 1) {
        const size_t wave = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 6;
        const size_t nwaves = ((size_t)gridDim.x * 256) >> 6;
        const unsigned lane = threadIdx.x & 63;
        for (size_t row = wave; row < outer; row += nwaves) {
            float s = 0.f;
            for (size_t d = lane; d < dim; d += 64)
                s += x[row * dim + d];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1)
                s += __shfl_xor(s, off);
            if (lane == 0)
                y[row] = s / (float)dim;
        }
        return;
    }
    size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t step = (size_t)gridDim.x * 256, total = outer * inner;
    for (; o < total; o += step) {
        const size_t ou = o / inner, i = o - ou * inner;
        const float *src = x + ou * dim * inner + i;
        float s = 0.f;
        for (size_t d = 0; d < dim; ++d)
            s += src[d * inner];
        y[o] = s / (float)dim;
    }
}

// Several outputs set to their bias (or zero) in one launch: blockIdx.y picks the
// output, y[o][c][i] = bias[c].
constexpr int kMaxFills = 24;
struct FillBatch {
    float *y[kMaxFills];
    const float *bias[kMaxFills];
    unsigned ch[kMaxFills], inner[kMaxFills];
    unsigned long long total[kMaxFills];
};

__global__ __launch_bounds__(256) void bias_fill_batch_kernel(FillBatch fb) {
    const int j = blockIdx.y;
    float *__restrict__ y = fb.y[j];
    const float *__restrict__ bias = fb.bias[j];
    const unsigned ch = fb.ch[j], inner = fb.inner[j];
    const size_t total = fb.total[j];
    const bool vec = inner % 4 == 0 && ((uintptr_t)y & 15) == 0;
    const size_t step = (size_t)gridDim.x * 256;
    if (vec) {
        for (size_t q = (size_t)blockIdx.x * 256 + threadIdx.x; q * 4 < total; q += step) {
            const float v = bias ? bias[(unsigned)((q * 4 / inner) % ch)] : 0.f;
            *reinterpret_cast<float4 *>(y + q * 4) = make_float4(v, v, v, v);
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += step)
            y[i] = bias ? bias[(unsigned)((i / inner) % ch)] : 0.f;
    }
}

__global__ __launch_bounds__(256) void bias_act_kernel(const float *__restrict__ x,
                                                       const float *__restrict__ bias,
                                                       float *__restrict__ y, size_t total,
                                                       unsigned ch, unsigned inner, int act) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t step = (size_t)gridDim.x * 256;
    for (; i < total; i += step) {
        unsigned c = (unsigned)((i / inner) % ch);
        float v = x[i] + (bias ? bias[c] : 0.f);
        y[i] = apply_act(v, act);
    }
}

// I: the index type, 32 bits when input and output have fewer than 2^31 elements (the three
// divisions of an output index are most of this kernel's instructions in 64 bits).
template <typename I>
__global__ __launch_bounds__(256) void pool2d_kernel(const float *__restrict__ x,
                                                     float *__restrict__ y, int nc, int h, int w,
                                                     int kh, int kw, int ph, int pw, int sh,
                                                     int sw, int dh, int dw, int oh, int ow,
                                                     int mode, float lo) {
    const I total = (I)nc * (I)oh * (I)ow;
    const I step = (I)gridDim.x * 256;
    for (I i = (I)blockIdx.x * 256 + threadIdx.x; i < total; i += step) {
        const int j = (int)(i % (I)ow);
        const I rest = i / (I)ow;
        const int ii = (int)(rest % (I)oh);
        const I plane = rest / (I)oh;
        const float *xp = x + plane * (I)h * (I)w;
        float acc = mode == 0 ? -INFINITY : 0.f;
        int taps = 0; // window positions inside the image: the divisor of an average
        for (int r = 0; r < kh; ++r) {
            int ih = ii * sh + r * dh - ph;
            if (ih < 0 || ih >= h)
                continue;
            for (int s = 0; s < kw; ++s) {
                int iw = j * sw + s * dw - pw;
                if (iw < 0 || iw >= w)
                    continue;
                float v = fmaxf(xp[ih * w + iw], lo); // lo = 0: ReLU on the way in
                acc = mode == 0 ? fmaxf(acc, v) : acc + v;
                ++taps;
            }
        }
        y[i] = mode == 0 ? acc : (taps ? acc / (float)taps : 0.f);
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Global average pooling: one wave per (n, c) plane.
__global__ __launch_bounds__(256) void global_avgpool_kernel(const float *__restrict__ x,
                                                             float *__restrict__ y, int nc,
                                                             int hw, float lo) {
    int plane = blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (plane >= nc)
        return;
    const float *xp = x + (size_t)plane * hw;
    float acc = 0.f;
    for (int i = lane; i < hw; i += 64)
        acc += fmaxf(xp[i], lo);
    acc = wave_sum(acc);
    if (lane == 0)
        y[plane] = acc / (float)hw;
}

// One wave per row. Rows of up to 64 * kRowRegs elements are read once into
// registers with all loads in flight (a row of BERT's 768 columns is 12 loads per
// lane; read three times one load after the other it costs 36 round trips);
// longer rows take the streaming variant. Both add in the same order.
constexpr int kRowRegs = 32;

template <bool RESIDENT>
__global__ __launch_bounds__(256) void softmax_kernel(const float *__restrict__ x,
                                                      float *__restrict__ y, size_t rows,
                                                      size_t cols) {
    size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (row >= rows)
        return;
    const float *xp = x + row * cols;
    float *yp = y + row * cols;
    if (RESIDENT) {
        float v[kRowRegs];
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i) {
            const size_t j = lane + 64 * (size_t)i;
            v[i] = j < cols ? xp[j] : -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i)
            mx = fmaxf(mx, v[i]);
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i) {
            const size_t j = lane + 64 * (size_t)i;
            v[i] = expf(v[i] - mx);
            if (j < cols)
                sum += v[i];
        }
        sum = wave_sum(sum);
        const float inv = 1.f / sum;
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i) {
            const size_t j = lane + 64 * (size_t)i;
            if (j < cols)
                yp[j] = v[i] * inv;
        }
        return;
    }
    float mx = -INFINITY;
    for (size_t j = lane; j < cols; j += 64)
        mx = fmaxf(mx, xp[j]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (size_t j = lane; j < cols; j += 64)
        sum += expf(xp[j] - mx);
    sum = wave_sum(sum);
    float inv = 1.f / sum;
    for (size_t j = lane; j < cols; j += 64)
        yp[j] = expf(xp[j] - mx) * inv;
}

// Rows of 256 * NV floats (NV <= 8), 16-byte aligned: a lane holds NV 16-byte words of the
// row, of gamma and of beta (a row of BERT's 768 columns is three loads per operand).
template <int NV>
__global__ __launch_bounds__(256) void layernorm_vec_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ gamma,
                                                            const float *__restrict__ beta,
                                                            float *__restrict__ y, size_t rows,
                                                            float eps) {
    constexpr int cols = 256 * NV;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows)
        return;
    const float4 *xp = reinterpret_cast<const float4 *>(x + row * cols);
    float4 *yp = reinterpret_cast<float4 *>(y + row * cols);
    float4 v[NV], gm[NV], bt[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        v[i] = xp[lane + 64 * i];
        gm[i] = gamma ? reinterpret_cast<const float4 *>(gamma)[lane + 64 * i]
                      : make_float4(1.f, 1.f, 1.f, 1.f);
        bt[i] = beta ? reinterpret_cast<const float4 *>(beta)[lane + 64 * i]
                     : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    const float mean = wave_sum(s) / (float)cols;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        v[i].x -= mean, v[i].y -= mean, v[i].z -= mean, v[i].w -= mean;
        q += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    }
    const float inv = rsqrtf(wave_sum(q) / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        float4 o;
        o.x = v[i].x * inv * gm[i].x + bt[i].x;
        o.y = v[i].y * inv * gm[i].y + bt[i].y;
        o.z = v[i].z * inv * gm[i].z + bt[i].z;
        o.w = v[i].w * inv * gm[i].w + bt[i].w;
        yp[lane + 64 * i] = o;
    }
}

template <bool RESIDENT>
__global__ __launch_bounds__(256) void layernorm_kernel(const float *__restrict__ x,
                                                        const float *__restrict__ gamma,
                                                        const float *__restrict__ beta,
                                                        float *__restrict__ y, size_t rows,
                                                        size_t cols, float eps) {
    size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    int lane = threadIdx.x & 63;
    if (row >= rows)
        return;
    const float *xp = x + row * cols;
    float *yp = y + row * cols;
    if (RESIDENT) {
        float v[kRowRegs], gm[kRowRegs], bt[kRowRegs];
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i) {
            const size_t j = lane + 64 * (size_t)i;
            const bool in = j < cols;
            v[i] = in ? xp[j] : 0.f;
            gm[i] = (in && gamma) ? gamma[j] : 1.f;
            bt[i] = (in && beta) ? beta[j] : 0.f;
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i)
            if (lane + 64 * (size_t)i < cols)
                s += v[i];
        const float mean = wave_sum(s) / (float)cols;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i)
            if (lane + 64 * (size_t)i < cols) {
                const float d = v[i] - mean;
                q += d * d;
            }
        const float inv = rsqrtf(wave_sum(q) / (float)cols + eps);
#pragma unroll
        for (int i = 0; i < kRowRegs; ++i) {
            const size_t j = lane + 64 * (size_t)i;
            if (j < cols) {
                float o = (v[i] - mean) * inv;
                if (gamma)
                    o *= gm[i];
                if (beta)
                    o += bt[i];
                yp[j] = o;
            }
        }
        return;
    }
    float s = 0.f;
    for (size_t j = lane; j < cols; j += 64)
        s += xp[j];
    float mean = wave_sum(s) / (float)cols;
    float v = 0.f;
    for (size_t j = lane; j < cols; j += 64) {
        float d = xp[j] - mean;
        v += d * d;
    }
    float inv = rsqrtf(wave_sum(v) / (float)cols + eps);
    for (size_t j = lane; j < cols; j += 64) {
        float o = (xp[j] - mean) * inv;
        if (gamma)
            o *= gamma[j];
        if (beta)
            o += beta[j];
        yp[j] = o;
    }
}

unsigned grid_for(size_t items) {
    size_t g = (items + 255) / 256;
    return (unsigned)std::min<size_t>(std::max<size_t>(g, 1), 1u << 20);
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

} // namespace

extern "C" {

int pet_hip_eltwise(int op, const float *const *ins, const size_t *sizes, int k, float *y,
                    size_t n, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (op != PET_HIP_ADD && op != PET_HIP_SUB && op != PET_HIP_MUL && op != PET_HIP_DIV)
        return set_error(PET_HIP_ERR_INVALID, "unknown element-wise op %d", op);
    if (k < 1 || k > kMaxEltIn || !ins || !sizes)
        return set_error(PET_HIP_ERR_INVALID, "element-wise ops take 1..%d inputs", kMaxEltIn);
    if ((op == PET_HIP_SUB || op == PET_HIP_DIV) && k != 2)
        return set_error(PET_HIP_ERR_INVALID, "Sub and Div are binary");
    if (n == 0)
        return PET_HIP_OK;
    if (!y)
        return set_error(PET_HIP_ERR_INVALID, "null output");
    if (n >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "element-wise ops are limited to 2^31 elements");
    EltParams p;
    memset(&p, 0, sizeof(p));
    p.k = k;
    p.op = op;
    p.n = n;
    // Div takes one element per thread: in the four-wide instance the compiler's
    // expansion of the division delivered elements 0 and 1 of every word into slots 2
    // and 3 and zeros into 0 and 1 (measured on gfx950 with ROCm 7.2).
    bool vec = (n % 4 == 0) && aligned16(y) && op != PET_HIP_DIV;
    for (int j = 0; j < k; ++j) {
        if (!ins[j] || sizes[j] == 0)
            return set_error(PET_HIP_ERR_INVALID, "input %d is empty", j);
        p.in[j] = ins[j];
        if (sizes[j] >= n) {
            p.size[j] = 0; // i % size == i
        } else {
            unsigned d = (unsigned)sizes[j];
            p.size[j] = d;
            if (d > 1) {
                unsigned l = 0;
                while ((1ull << l) < d)
                    ++l;
                unsigned pw = 31 + l;
                p.mul[j] = (unsigned)(((1ull << pw) + d - 1) / d);
                p.shift[j] = pw - 32;
            }
            if (d != 1 && d % 4)
                vec = false;
        }
        if (!aligned16(ins[j]))
            vec = false;
    }
    if (vec)
        hipLaunchKernelGGL(eltwise_kernel<4>, dim3(grid_for(n / 4)), dim3(256), 0,
                           as_stream(stream), p, y);
    else
        hipLaunchKernelGGL(eltwise_kernel<1>, dim3(grid_for(n)), dim3(256), 0, as_stream(stream),
                           p, y);
    return check_launch("eltwise_kernel");
}

int pet_hip_activation(const float *x, float *y, size_t n, int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (act < PET_HIP_ACT_NONE || act > PET_HIP_ACT_GELU)
        return set_error(PET_HIP_ERR_INVALID, "unknown activation %d", act);
    if (n == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (n % 4 == 0 && aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(activation_kernel<4>, dim3(grid_for(n / 4)), dim3(256), 0,
                           as_stream(stream), x, y, n, act);
    else
        hipLaunchKernelGGL(activation_kernel<1>, dim3(grid_for(n)), dim3(256), 0,
                           as_stream(stream), x, y, n, act);
    return check_launch("activation_kernel");
}

int pet_hip_pow(const float *x, float *y, size_t n, int pow, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (pow > 1024)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "power %d is beyond 1024", pow);
    if (n == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (n % 4 == 0 && aligned16(x) && aligned16(y))
        hipLaunchKernelGGL(pow_kernel<4>, dim3(grid_for(n / 4)), dim3(256), 0, as_stream(stream), x,
                           y, n, pow);
    else
        hipLaunchKernelGGL(pow_kernel<1>, dim3(grid_for(n)), dim3(256), 0, as_stream(stream), x, y,
                           n, pow);
    return check_launch("pow_kernel");
}

int pet_hip_batchnorm(const float *x, const float *scale, const float *bias, const float *mean,
                      const float *var, float *y, size_t outer, size_t ch, size_t inner, float eps,
                      pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    const size_t rows = outer * ch;
    if (rows == 0 || inner == 0)
        return PET_HIP_OK;
    if (!x || !y || !scale || !bias || !mean || !var)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (ch >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "too many channels");
    const int vec = inner % 4 == 0 && aligned16(x) && aligned16(y);
    const unsigned grid = (unsigned)std::min<size_t>(rows, 65536);
    hipLaunchKernelGGL(batchnorm_kernel, dim3(grid), dim3(256), 0, as_stream(stream), x, scale,
                       bias, mean, var, y, rows, (unsigned)ch, inner, eps, vec);
    return check_launch("batchnorm_kernel");
}

int pet_hip_gather(const float *x, const void *indices, int index_is_float, float *y, size_t pre,
                   size_t dim, size_t post, size_t nidx, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    const size_t total = nidx * pre * post;
    if (total == 0)
        return PET_HIP_OK;
    if (!x || !indices || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (dim == 0)
        return set_error(PET_HIP_ERR_INVALID, "gather along an empty axis");
    if (total >= (1ull << 40) || dim >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "gather is limited to 2^40 outputs");
    if (index_is_float)
        hipLaunchKernelGGL(gather_kernel<true>, dim3(grid_for(total)), dim3(256), 0,
                           as_stream(stream), x, indices, y, total, pre, (long long)dim, post);
    else
        hipLaunchKernelGGL(gather_kernel<false>, dim3(grid_for(total)), dim3(256), 0,
                           as_stream(stream), x, indices, y, total, pre, (long long)dim, post);
    return check_launch("gather_kernel");
}

int pet_hip_reduce_mean(const float *x, float *y, size_t outer, size_t dim, size_t inner,
                        pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (outer * inner == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (dim == 0)
        return set_error(PET_HIP_ERR_INVALID, "mean over an empty axis");
    const size_t threads = inner == 1 ? outer * 64 : outer * inner;
    hipLaunchKernelGGL(reduce_mean_kernel, dim3(grid_for(threads)), dim3(256), 0, as_stream(stream),
                       x, y, outer, dim, inner);
    return check_launch("reduce_mean_kernel");
}

int pet_hip_bias_fill_batch(const pet_hip_fill *fills, int count, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (count < 0 || (count > 0 && !fills))
        return set_error(PET_HIP_ERR_INVALID, "bad fill list");
    for (int base = 0; base < count; base += kMaxFills) {
        FillBatch fb;
        memset(&fb, 0, sizeof(fb));
        int nb = 0;
        size_t most = 0;
        for (int i = base; i < count && i < base + kMaxFills; ++i) {
            const pet_hip_fill &f = fills[i];
            const size_t total = f.outer * f.ch * f.inner;
            if (total == 0)
                continue;
            if (!f.y)
                return set_error(PET_HIP_ERR_INVALID, "fill %d has no output", i);
            if (f.ch >= (1ull << 32) || f.inner >= (1ull << 32))
                return set_error(PET_HIP_ERR_UNSUPPORTED, "fill %d is too large", i);
            fb.y[nb] = f.y;
            fb.bias[nb] = f.bias;
            fb.ch[nb] = (unsigned)f.ch;
            fb.inner[nb] = (unsigned)f.inner;
            fb.total[nb] = total;
            most = std::max(most, total);
            ++nb;
        }
        if (nb == 0)
            continue;
        const unsigned gx = (unsigned)std::min<size_t>((most / 4 + 255) / 256 + 1, 1024);
        hipLaunchKernelGGL(bias_fill_batch_kernel, dim3(gx, nb), dim3(256), 0, as_stream(stream),
                           fb);
        int rc = check_launch("bias_fill_batch_kernel");
        if (rc)
            return rc;
    }
    return PET_HIP_OK;
}

int pet_hip_bias_act(const float *x, const float *bias, float *y, size_t outer, size_t ch,
                     size_t inner, int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (act < PET_HIP_ACT_NONE || act > PET_HIP_ACT_GELU)
        return set_error(PET_HIP_ERR_INVALID, "unknown activation %d", act);
    size_t total = outer * ch * inner;
    if (total == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if (ch >= (1ull << 31) || inner >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "bias_act dims too large");
    hipLaunchKernelGGL(bias_act_kernel, dim3(grid_for(total)), dim3(256), 0, as_stream(stream), x,
                       bias, y, total, (unsigned)ch, (unsigned)inner, act);
    return check_launch("bias_act_kernel");
}

int pet_hip_pool2d(const float *x, float *y, int n, int c, int h, int w, int kh, int kw, int ph,
                   int pw, int sh, int sw, int dh, int dw, int mode, pet_hip_stream_t stream) {
    return pet_hip_pool2d_ex(x, y, n, c, h, w, kh, kw, ph, pw, sh, sw, dh, dw, mode, 0, stream);
}

int pet_hip_pool2d_ex(const float *x, float *y, int n, int c, int h, int w, int kh, int kw, int ph,
                      int pw, int sh, int sw, int dh, int dw, int mode, unsigned flags,
                      pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (flags & ~(unsigned)PET_HIP_CALL_X_RELU)
        return set_error(PET_HIP_ERR_INVALID, "pooling takes PET_HIP_CALL_X_RELU only");
    const float lo = (flags & PET_HIP_CALL_X_RELU) ? 0.f : -INFINITY;
    if (n < 0 || c < 0 || h <= 0 || w <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 ||
        dh <= 0 || dw <= 0 || ph < 0 || pw < 0 || (mode != 0 && mode != 1))
        return set_error(PET_HIP_ERR_INVALID, "bad pooling arguments");
    int oh = (h + 2 * ph - dh * (kh - 1) - 1) / sh + 1;
    int ow = (w + 2 * pw - dw * (kw - 1) - 1) / sw + 1;
    if (oh <= 0 || ow <= 0)
        return set_error(PET_HIP_ERR_INVALID, "pooling window larger than the image");
    size_t total = (size_t)n * c * oh * ow;
    if (total == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if ((long long)n * c >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "pooling over 2^31 planes or more");
    if (mode == 1 && kh == h && kw == w && ph == 0 && pw == 0 && dh == 1 && dw == 1) {
        int nc = n * c;
        hipLaunchKernelGGL(global_avgpool_kernel, dim3((nc + 3) / 4), dim3(256), 0,
                           as_stream(stream), x, y, nc, h * w, lo);
        return check_launch("global_avgpool_kernel");
    }
    if ((size_t)n * c * h * w < (1ull << 31) && total < (1ull << 31))
        hipLaunchKernelGGL(pool2d_kernel<unsigned>, dim3(grid_for(total)), dim3(256), 0,
                           as_stream(stream), x, y, n * c, h, w, kh, kw, ph, pw, sh, sw, dh, dw,
                           oh, ow, mode, lo);
    else
        hipLaunchKernelGGL(pool2d_kernel<size_t>, dim3(grid_for(total)), dim3(256), 0,
                           as_stream(stream), x, y, n * c, h, w, kh, kw, ph, pw, sh, sw, dh, dw,
                           oh, ow, mode, lo);
    return check_launch("pool2d_kernel");
}

int pet_hip_softmax(const float *x, float *y, size_t rows, size_t cols, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (rows == 0 || cols == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if ((rows + 3) / 4 >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "too many rows");
    if (cols <= 64 * (size_t)kRowRegs)
        hipLaunchKernelGGL(softmax_kernel<true>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                           as_stream(stream), x, y, rows, cols);
    else
        hipLaunchKernelGGL(softmax_kernel<false>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                           as_stream(stream), x, y, rows, cols);
    return check_launch("softmax_kernel");
}

int pet_hip_layernorm(const float *x, const float *gamma, const float *beta, float *y, size_t rows,
                      size_t cols, float eps, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (rows == 0 || cols == 0)
        return PET_HIP_OK;
    if (!x || !y)
        return set_error(PET_HIP_ERR_INVALID, "null pointer");
    if ((rows + 3) / 4 >= (1ull << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "too many rows");
    const bool aligned = ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)gamma) | ((uintptr_t)beta)) & 15) == 0;
    const dim3 grid((unsigned)((rows + 3) / 4));
    if (aligned && cols % 256 == 0 && cols <= 2048) {
        hipStream_t st = as_stream(stream);
        switch (cols / 256) {
#define PET_LN_CASE(NV)                                                                            \
    case NV:                                                                                       \
        hipLaunchKernelGGL(layernorm_vec_kernel<NV>, grid, dim3(256), 0, st, x, gamma, beta, y,    \
                           rows, eps);                                                             \
        break;
            PET_LN_CASE(1)
            PET_LN_CASE(2)
            PET_LN_CASE(3)
            PET_LN_CASE(4)
            PET_LN_CASE(5)
            PET_LN_CASE(6)
            PET_LN_CASE(7)
            PET_LN_CASE(8)
#undef PET_LN_CASE
        }
        return check_launch("layernorm_vec_kernel");
    }
    if (cols <= 64 * (size_t)kRowRegs)
        hipLaunchKernelGGL(layernorm_kernel<true>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                           as_stream(stream), x, gamma, beta, y, rows, cols, eps);
    else
        hipLaunchKernelGGL(layernorm_kernel<false>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0,
                           as_stream(stream), x, gamma, beta, y, rows, cols, eps);
    return check_launch("layernorm_kernel");
}

} // extern "C"
