// Transposed convolution (ConvTransOp, src/Graph/operator.cc:932-983): input NHWF,
// weight RSFC, output NHWC, fp32 MFMA.
//
// An output row hh takes input row (hh + rr*dh - (r-ph-1)) / sh for the taps rr where
// that division is exact, so which taps contribute depends only on hh mod sh (and ww mod
// sw). The kernel therefore works one residue class ("phase") at a time: inside a phase
// every output pixel uses the same taps, the input pixel moves with the output pixel, and
// the whole thing is a dense GEMM per tap:
//     y[pixel][c] += x[pixel shifted by the tap][f] * w[r-1-rr][s-1-ss][f][c].
// M = the pixels of the phase (batch folded in), N = output channels, K = f per tap.
// NHWF / RSFC put K contiguous for the pixel operand and N contiguous for the filter
// operand, which is exactly how v_mfma_f32_32x32x2_f32 wants its lanes fed: a lane holds
// one pixel (16-byte loads along f) and one channel (coalesced dword loads across lanes);
// no LDS staging. A wave owns 32 pixels x 32*TN channels, a workgroup four pixel tiles.
#include "mfma_common.h"

using namespace pet;
using namespace pet::mfma;

namespace {

struct ConvTransParams {
    const float *x, *w, *bias;
    float *y;
    int N, H, W, F, R, S, C;
    int ph, pw, sh, sw, dh, dw;
    int OH, OW;
    int ah, aw; // taps rr > R - ah (ss > S - aw) are left out, as the reference does
    int act;
};

template <int TN, bool VEC>
__global__ __launch_bounds__(256) void conv_trans_kernel(ConvTransParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hk = lane >> 5;
    const int qh = blockIdx.z / p.sw, qw = blockIdx.z - qh * p.sw;
    // this phase's pixel grid: output rows qh, qh + sh, ...
    const int OHq = qh < p.OH ? (p.OH - qh + p.sh - 1) / p.sh : 0;
    const int OWq = qw < p.OW ? (p.OW - qw + p.sw - 1) / p.sw : 0;
    const int npix = p.N * OHq * OWq;
    const int pix0 = (blockIdx.x * 4 + wave) * 32;
    if (pix0 >= npix)
        return;
    const int c0 = blockIdx.y * (32 * TN);

    // this lane's pixel (rows past the end repeat the last pixel and are not stored)
    const int pix = min(pix0 + l32, npix - 1);
    const int n = pix / (OHq * OWq);
    const int rem = pix - n * (OHq * OWq);
    const int pi = rem / OWq, pj = rem - pi * OWq;
    const int ybase = pix0 + l32 < npix
                          ? ((n * p.OH + qh + pi * p.sh) * p.OW + qw + pj * p.sw) * p.C
                          : -1;

    floatx16 acc[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[tn][r] = 0.f;

    int cc[TN];
    bool cok[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        cc[tn] = min(c0 + tn * 32 + l32, p.C - 1);
        cok[tn] = c0 + tn * 32 + l32 < p.C;
    }

    for (int rr = 0; rr < p.R; ++rr) {
        if (p.R - p.ah < rr)
            continue;
        const int th = qh + rr * p.dh - (p.R - p.ph - 1);
        if (th % p.sh != 0)
            continue;
        const int ih = th / p.sh + pi;
        for (int ss = 0; ss < p.S; ++ss) {
            if (p.S - p.aw < ss)
                continue;
            const int tw = qw + ss * p.dw - (p.S - p.pw - 1);
            if (tw % p.sw != 0)
                continue;
            const int iw = tw / p.sw + pj;
            const bool inside = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            const float *xp =
                p.x + (size_t)((n * p.H + (inside ? ih : 0)) * p.W + (inside ? iw : 0)) * p.F;
            const float *wp = p.w + (size_t)((p.R - 1 - rr) * p.S + (p.S - 1 - ss)) * p.F * p.C;
            for (int f0 = 0; f0 < p.F; f0 += 8) {
                const int fk = f0 + hk * 4; // this half-wave's four k values
                float a[4], b[TN][4];
                if (VEC) {
                    float4 v = inside ? *reinterpret_cast<const float4 *>(xp + fk)
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
                    a[0] = v.x;
                    a[1] = v.y;
                    a[2] = v.z;
                    a[3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        a[j] = (inside && fk + j < p.F) ? xp[fk + j] : 0.f;
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn) {
                        const bool ok = cok[tn] && (VEC || fk + j < p.F);
                        b[tn][j] = ok ? wp[(size_t)(fk + j) * p.C + cc[tn]] : 0.f;
                    }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
                        acc[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[tn][j], acc[tn], 0,
                                                                       0, 0);
            }
        }
    }

    // accumulator register r of a lane is pixel row (r/4)*8 + hk*4 + r%4, channel l32
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = (r / 4) * 8 + hk * 4 + (r % 4);
        const int yo = __shfl(ybase, m);
        if (yo < 0)
            continue;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            if (!cok[tn])
                continue;
            float v = acc[tn][r];
            if (p.bias)
                v += p.bias[cc[tn]];
            p.y[(size_t)yo + cc[tn]] = apply_act(v, p.act);
        }
    }
}

} // namespace

extern "C" {

int pet_hip_conv_trans_out_dim(int i, int k, int p, int s, int d, int op) {
    return (i - 1) * s - 2 * p + d * (k - 1) + op + 1;
}

int pet_hip_conv_trans_f32(const float *x, const float *w, const float *bias, float *y, int n,
                           int h, int wd, int f, int r, int s, int c, int ph, int pw, int sh,
                           int sw, int dh, int dw, int oph, int opw, int act,
                           pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!x || !w || !y)
        return set_error(PET_HIP_ERR_INVALID, "conv_trans: null operand");
    if (n <= 0 || h <= 0 || wd <= 0 || f <= 0 || r <= 0 || s <= 0 || c <= 0 || sh <= 0 ||
        sw <= 0 || dh <= 0 || dw <= 0 || ph < 0 || pw < 0 || oph < 0 || opw < 0)
        return set_error(PET_HIP_ERR_INVALID, "conv_trans: bad shape or parameter");
    ConvTransParams p;
    p.x = x;
    p.w = w;
    p.bias = bias;
    p.y = y;
    p.N = n;
    p.H = h;
    p.W = wd;
    p.F = f;
    p.R = r;
    p.S = s;
    p.C = c;
    p.ph = ph;
    p.pw = pw;
    p.sh = sh;
    p.sw = sw;
    p.dh = dh;
    p.dw = dw;
    p.OH = pet_hip_conv_trans_out_dim(h, r, ph, sh, dh, oph);
    p.OW = pet_hip_conv_trans_out_dim(wd, s, pw, sw, dw, opw);
    p.ah = (h + 2 * ph - r) % sh;
    p.aw = (wd + 2 * pw - s) % sw;
    p.act = act;
    if (p.OH <= 0 || p.OW <= 0)
        return set_error(PET_HIP_ERR_INVALID, "conv_trans: empty output %d x %d", p.OH, p.OW);
    const long long xin = (long long)n * h * wd * f, yout = (long long)n * p.OH * p.OW * c,
                    wel = (long long)r * s * f * c;
    if (xin >= (1ll << 31) || yout >= (1ll << 31) || wel >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: tensors of 2^31 elements or more");
    if (sh * sw > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: stride %d x %d", sh, sw);
    const int tn = c > 32 ? 2 : 1;
    // the largest phase is phase (0, 0)
    const long long maxpix = (long long)n * ((p.OH + sh - 1) / sh) * ((p.OW + sw - 1) / sw);
    dim3 grid((unsigned)((maxpix + 127) / 128), (unsigned)((c + 32 * tn - 1) / (32 * tn)),
              (unsigned)(sh * sw));
    if (grid.y > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: %d output channels", c);
    const bool vec = f % 8 == 0 && ((uintptr_t)x & 15) == 0;
    hipStream_t st = as_stream(stream);
    if (tn == 2) {
        if (vec)
            hipLaunchKernelGGL((conv_trans_kernel<2, true>), grid, dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL((conv_trans_kernel<2, false>), grid, dim3(256), 0, st, p);
    } else {
        if (vec)
            hipLaunchKernelGGL((conv_trans_kernel<1, true>), grid, dim3(256), 0, st, p);
        else
            hipLaunchKernelGGL((conv_trans_kernel<1, false>), grid, dim3(256), 0, st, p);
    }
    return check_launch("conv_trans_kernel");
}

} // extern "C"
