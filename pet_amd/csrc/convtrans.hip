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
#include <algorithm>
#include <type_traits>

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
    int PT, KW; // pixel tiles and feature shares per workgroup
    int nfast;  // pixel numbering, see the kernel
    int KS;     // workgroups sharing a tile's taps (their sums meet in y as float atomics)
    int act;
};

// A workgroup is PT pixel tiles x KW shares of the feature axis (PT * KW waves). With many
// pixel tiles KW is 1 and a wave stores its tile itself; a layer with few pixels and many
// features (the first layers of a generator network: 2x2 pixels, 448 features) would leave
// one wave per tile walking all of K with nothing to hide its load latency, so there the
// feature axis is dealt to up to 16 waves, which add their tiles in LDS in wave order
// (results do not depend on timing) and share the stores.
template <int TN, bool VEC, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 1024 : 256) void conv_trans_kernel(ConvTransParams p) {
    static_assert(!SPLIT || TN == 1, "the shared form is 32 channels wide");
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hk = lane >> 5;
    const int pt = SPLIT ? wave % p.PT : wave, kw = SPLIT ? wave / p.PT : 0;
    const int qh = blockIdx.z / p.sw, qw = blockIdx.z - qh * p.sw;
    // this phase's pixel grid: output rows qh, qh + sh, ...
    const int OHq = qh < p.OH ? (p.OH - qh + p.sh - 1) / p.sh : 0;
    const int OWq = qw < p.OW ? (p.OW - qw + p.sw - 1) / p.sw : 0;
    const int npix = p.N * OHq * OWq;
    const int ks = SPLIT ? (int)(blockIdx.x % (unsigned)p.KS) : 0; // this workgroup's taps
    const int pix0 = ((SPLIT ? blockIdx.x / (unsigned)p.KS : blockIdx.x) * p.PT + pt) * 32;
    const bool active = pix0 < npix;
    if (!SPLIT && !active)
        return;
    const int c0 = blockIdx.y * (32 * TN);

    // this lane's pixel (rows past the end repeat the last pixel and are not stored)
    const int pix = max(min(pix0 + l32, npix - 1), 0);
    const int plane = max(OHq * OWq, 1);
    // pixels of a phase are numbered image-major, or (nfast) with the image number running
    // fastest: with 32 images or more the lanes of a tile then sit at one output position and
    // agree on which taps reach the input at all
    const int n = p.nfast ? pix % p.N : pix / plane;
    const int rem = p.nfast ? pix / p.N : pix - n * plane;
    const int pi = rem / max(OWq, 1), pj = rem - pi * max(OWq, 1);
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

    // this wave's share of the feature axis, in chunks of 8 features
    const int nch = (p.F + 7) / 8;
    const int ch_lo = SPLIT ? kw * nch / p.KW : 0, ch_hi = SPLIT ? (kw + 1) * nch / p.KW : nch;

    for (int rr = 0; rr < p.R && active; ++rr) {
        if (p.R - p.ah < rr)
            continue;
        const int th = qh + rr * p.dh - (p.R - p.ph - 1);
        if (th % p.sh != 0)
            continue;
        const int ih = th / p.sh + pi;
        for (int ss = 0; ss < p.S; ++ss) {
            // (every sh-th row and sw-th column of taps reaches a phase: numbering them by
            // rr / sh and ss / sw deals a phase's taps evenly)
            if (p.S - p.aw < ss ||
                (SPLIT && ((rr / p.sh) * ((p.S + p.sw - 1) / p.sw) + ss / p.sw) % p.KS != ks))
                continue;
            const int tw = qw + ss * p.dw - (p.S - p.pw - 1);
            if (tw % p.sw != 0)
                continue;
            const int iw = tw / p.sw + pj;
            const bool inside = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            if (__builtin_amdgcn_ballot_w64(inside) == 0)
                continue; // no lane of the wave has an input pixel under this tap
            const float *xp =
                p.x + (size_t)((n * p.H + (inside ? ih : 0)) * p.W + (inside ? iw : 0)) * p.F;
            const float *wp = p.w + (size_t)((p.R - 1 - rr) * p.S + (p.S - 1 - ss)) * p.F * p.C;
            // U chunks per trip: all their loads are issued before the first MFMA
            auto trip = [&](int ch, auto ucount) {
                constexpr int U = decltype(ucount)::value;
                float a[U][4], b[U][TN][4];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int fk = (ch + u) * 8 + hk * 4; // this half-wave's four k values
                    // VEC: F is a multiple of 4, so the four are all inside or all outside
                    const bool fin = fk < p.F;
                    if (VEC) {
                        float4 v = inside && fin ? *reinterpret_cast<const float4 *>(xp + fk)
                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
                        a[u][0] = v.x;
                        a[u][1] = v.y;
                        a[u][2] = v.z;
                        a[u][3] = v.w;
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            a[u][j] = (inside && fk + j < p.F) ? xp[fk + j] : 0.f;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn) {
                            const bool ok = cok[tn] && (VEC ? fin : fk + j < p.F);
                            b[u][tn][j] = ok ? wp[(size_t)(fk + j) * p.C + cc[tn]] : 0.f;
                        }
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int tn = 0; tn < TN; ++tn)
                            acc[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][j], b[u][tn][j],
                                                                           acc[tn], 0, 0, 0);
            };
            int ch = ch_lo;
            for (; ch + 4 <= ch_hi; ch += 4)
                trip(ch, std::integral_constant<int, 4>{});
            for (; ch < ch_hi; ++ch)
                trip(ch, std::integral_constant<int, 1>{});
        }
    }

    if (!SPLIT) {
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
        return;
    }

    // per pixel tile: [32 rows][32 * TN channels] sums, then the 32 row offsets
    constexpr int TW = 32 * TN;
    float *tile = lds + pt * (32 * TW + 32);
    int *yoff = reinterpret_cast<int *>(tile + 32 * TW);
    if (kw == 0 && hk == 0)
        yoff[l32] = ybase;
    for (int w = 0; w < p.KW; ++w) {
        if (kw == w && active) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = (r / 4) * 8 + hk * 4 + (r % 4);
                    float *dst = tile + m * TW + tn * 32 + l32;
                    *dst = w == 0 ? acc[tn][r] : *dst + acc[tn][r];
                }
        }
        __syncthreads();
    }
    if (!active)
        return;
    // the KW waves of a tile share its rows; a lane stores channel c0 + j of a row
    for (int e = kw * 64 + lane; e < 32 * TW; e += p.KW * 64) {
        const int m = e / TW, j = e - m * TW;
        const int yo = yoff[m];
        if (yo < 0 || c0 + j >= p.C)
            continue;
        float v = tile[e];
        if (p.KS > 1) { // y holds the bias already; the activation follows in a launch of its own
            unsafeAtomicAdd(p.y + (size_t)yo + c0 + j, v);
            continue;
        }
        if (p.bias)
            v += p.bias[c0 + j];
        p.y[(size_t)yo + c0 + j] = apply_act(v, p.act);
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
    if (n < 0 || h <= 0 || wd <= 0 || f <= 0 || r <= 0 || s <= 0 || c <= 0 || sh <= 0 ||
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
    p.nfast = n >= 32;
    if (p.OH <= 0 || p.OW <= 0)
        return set_error(PET_HIP_ERR_INVALID, "conv_trans: empty output %d x %d", p.OH, p.OW);
    if (n == 0)
        return PET_HIP_OK; // an empty batch: nothing to compute, as in the convolutions
    if (!x || !w || !y)
        return set_error(PET_HIP_ERR_INVALID, "conv_trans: null operand");
    const long long xin = (long long)n * h * wd * f, yout = (long long)n * p.OH * p.OW * c,
                    wel = (long long)r * s * f * c;
    if (xin >= (1ll << 31) || yout >= (1ll << 31) || wel >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: tensors of 2^31 elements or more");
    if (sh * sw > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: stride %d x %d", sh, sw);
    // the largest phase is phase (0, 0)
    const long long maxpix = (long long)n * ((p.OH + sh - 1) / sh) * ((p.OW + sw - 1) / sw);
    const long long tiles = (maxpix + 31) / 32;
    int tn = c > 32 ? 2 : 1;
    if (tn == 2 && tiles * ((c + 63) / 64) * sh * sw < 1024)
        tn = 1; // few tiles: narrower ones reach more CUs (and the shared form is 32 wide)
    const long long waves = tiles * ((c + 32 * tn - 1) / (32 * tn)) * sh * sw;
    const int nch = (f + 7) / 8;
    p.PT = (int)(tiles < 4 ? tiles : 4);
    p.KW = 1;
    if (waves < 1024) {
        long long want = (1024 + waves - 1) / waves;
        want = want < 16 / p.PT ? want : 16 / p.PT;
        want = want < nch / 4 ? want : nch / 4; // at least four chunks per wave
        p.KW = want > 1 ? (int)want : 1;
    }
    const bool split = p.KW > 1;
    if (!split)
        p.PT = 4;
    // still far from a wave per SIMD (2x2 pixels, 448 features): the taps are dealt to KS
    // workgroups as well, whose sums meet in y as float atomics: y is initialised with the
    // bias before and activated after. Not in reproducible mode.
    p.KS = 1;
    if (split && !deterministic()) {
        const long long now = waves * p.KW;
        const int taps = ((r + sh - 1) / sh) * ((s + sw - 1) / sw); // per phase
        int ks = (int)std::min<long long>((1024 + now - 1) / now, 16);
        ks = std::min(ks, taps / 2);
        if (ks >= 2)
            p.KS = ks;
    }
    dim3 grid((unsigned)((tiles + p.PT - 1) / p.PT) * (unsigned)p.KS,
              (unsigned)((c + 32 * tn - 1) / (32 * tn)), (unsigned)(sh * sw));
    if (grid.y > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "conv_trans: %d output channels", c);
    const bool vec = f % 4 == 0 && ((uintptr_t)x & 15) == 0;
    hipStream_t st = as_stream(stream);
    if (p.KS > 1) {
        pet_hip_fill fill{y, bias, (size_t)n * p.OH * p.OW, (size_t)c, 1};
        if (int rc = pet_hip_bias_fill_batch(&fill, 1, stream))
            return rc;
    }
    const dim3 block(64u * p.PT * p.KW);
    const size_t lds = split ? sizeof(float) * p.PT * (32 * 32 * tn + 32) : 0;
    auto launch = [&](auto tn_, auto vec_) {
        constexpr int TN_ = decltype(tn_)::value;
        constexpr bool VEC_ = decltype(vec_)::value;
        if (split && TN_ == 1)
            hipLaunchKernelGGL((conv_trans_kernel<1, VEC_, true>), grid, block, lds, st, p);
        else
            hipLaunchKernelGGL((conv_trans_kernel<TN_, VEC_, false>), grid, block, lds, st, p);
    };
    using two = std::integral_constant<int, 2>;
    using one = std::integral_constant<int, 1>;
    if (tn == 2)
        vec ? launch(two{}, std::true_type{}) : launch(two{}, std::false_type{});
    else
        vec ? launch(one{}, std::true_type{}) : launch(one{}, std::false_type{});
    if (int rc = check_launch("conv_trans_kernel"))
        return rc;
    if (p.KS > 1 && act != PET_HIP_ACT_NONE)
        return pet_hip_activation(y, y, (size_t)yout, act, stream);
    return PET_HIP_OK;
}

} // extern "C"
