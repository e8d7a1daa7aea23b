// Band matrix products of sliding-window attention, fp32 MFMA:
//   G2BMM  C[b,i,j] = sum_k A[b,i,k] * B[b, i + d*(j-w), k]       (general x general -> band)
//   GBMML  C[b,i,n] = sum_j A[b,i,j] * B[b, i + d*j - d*w, n]     (band x general -> general)
// with j in [0, 2w] and rows of B outside [0, m) read as zero; the definitions are the
// expressions the reference's search works on (Sg2bmmPattern / LongformerGBMMPattern,
// src/nnet/iterator_table.cc:596-630). The reference runs them through two generated
// kernels fixed to m = 10000, k = 64, w = 1000, d in {1, 4} (include/custom_ops.cuh:
// 3538-3559); these kernels take any shape.
//
// Rows i and i + d*(j-w) are congruent modulo d, so each residue class rho of rows is a
// problem with dilation 1 on the rows rho, rho + d, ...: row i' of the class meets row r'
// of the class at band column j = r' - i' + w.
//  * G2BMM computes dense 32x32 tiles T[i'][r'] = A[i'] . B[r'] (both operands contiguous
//    along k: 16-byte loads per lane) and stores the part of each tile that lies in the
//    band: a lane's 32 columns r' are 32 consecutive j of one output row, a coalesced store.
//  * GBMML is a GEMM whose K axis runs over r' in [i0' - w, i0' + 31 + w]: the band operand
//    is read per lane along j (contiguous, zero outside the band), the general operand
//    across lanes along n (coalesced).
#include "mfma_common.h"

using namespace pet;
using namespace pet::mfma;

namespace {

struct BandParams {
    const float *A, *B;
    float *C;
    int bs, m, k, w, d, n; // k: G2BMM feature length; n: GBMML output columns
    int mc;                // rows per residue class, rounded up: ceil(m / d)
    int rtiles;            // G2BMM: column tiles per row block
};

// grid: x = r' tile, y = i' block, z = batch * d + rho
__global__ __launch_bounds__(64) void g2bmm_kernel(BandParams p) {
    const int lane = threadIdx.x;
    const int l32 = lane & 31, hk = lane >> 5;
    const int b = blockIdx.z / p.d, rho = blockIdx.z - b * p.d;
    const int rows = rho < p.m ? (p.m - rho + p.d - 1) / p.d : 0; // rows of this class
    const int i0 = blockIdx.y * 32;
    if (i0 >= rows)
        return;
    // first column tile that can touch the band of rows i0 .. i0 + 31
    const int rfirst = i0 - p.w;
    const int r0 = rfirst + (int)blockIdx.x * 32;
    if (r0 > i0 + 31 + p.w)
        return;
    const int ia = min(i0 + l32, rows - 1);
    const int rb = r0 + l32;
    const bool rok = rb >= 0 && rb < rows;
    const float *ap = p.A + ((size_t)b * p.m + rho + (size_t)ia * p.d) * p.k;
    const float *bp = p.B + ((size_t)b * p.m + rho + (size_t)(rok ? rb : 0) * p.d) * p.k;
    const bool vec = p.k % 8 == 0 && ((((uintptr_t)p.A) | ((uintptr_t)p.B)) & 15) == 0;
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        acc[r] = 0.f;
    for (int k0 = 0; k0 < p.k; k0 += 8) {
        const int kk = k0 + hk * 4;
        float a[4], bv[4];
        if (vec) {
            const float4 va = *reinterpret_cast<const float4 *>(ap + kk);
            const float4 vb = rok ? *reinterpret_cast<const float4 *>(bp + kk)
                                  : make_float4(0.f, 0.f, 0.f, 0.f);
            a[0] = va.x, a[1] = va.y, a[2] = va.z, a[3] = va.w;
            bv[0] = vb.x, bv[1] = vb.y, bv[2] = vb.z, bv[3] = vb.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a[j] = kk + j < p.k ? ap[kk + j] : 0.f;
                bv[j] = (rok && kk + j < p.k) ? bp[kk + j] : 0.f;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv[j], acc, 0, 0, 0);
    }
    // register r: row i0 + (r/4)*8 + hk*4 + r%4, column r0 + l32 -> band column j
    const int band = 2 * p.w + 1;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int il = i0 + (r / 4) * 8 + hk * 4 + (r % 4);
        const int j = rb - il + p.w;
        if (il < rows && j >= 0 && j < band)
            p.C[((size_t)b * p.m + rho + (size_t)il * p.d) * band + j] = acc[r]; // 0 when !rok
    }
}

// grid: x = n tile (32 * TN columns), y = i' block, z = batch * d + rho
template <int TN>
__global__ __launch_bounds__(64) void gbmml_kernel(BandParams p) {
    const int lane = threadIdx.x;
    const int l32 = lane & 31, hk = lane >> 5;
    const int b = blockIdx.z / p.d, rho = blockIdx.z - b * p.d;
    const int rows = rho < p.m ? (p.m - rho + p.d - 1) / p.d : 0;
    const int i0 = blockIdx.y * 32;
    if (i0 >= rows)
        return;
    const int n0 = blockIdx.x * (32 * TN);
    const int band = 2 * p.w + 1;
    const int ia = min(i0 + l32, rows - 1);
    const float *ap = p.A + ((size_t)b * p.m + rho + (size_t)ia * p.d) * band;
    int cn[TN];
    bool nok[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        cn[tn] = min(n0 + tn * 32 + l32, p.n - 1);
        nok[tn] = n0 + tn * 32 + l32 < p.n;
    }
    floatx16 acc[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[tn][r] = 0.f;
    // K axis: class rows r' that any of the 32 output rows can reach
    const int rlo = max(i0 - p.w, 0), rhi = min(i0 + 31 + p.w, rows - 1);
    for (int r0 = rlo; r0 <= rhi; r0 += 8) {
        float a[4], bv[TN][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int rr = r0 + hk * 4 + j;
            const int jj = rr - ia + p.w; // band column of (row ia, class row rr)
            const bool rin = rr <= rhi;
            a[j] = (rin && jj >= 0 && jj < band) ? ap[jj] : 0.f;
            const float *bp = p.B + ((size_t)b * p.m + rho + (size_t)(rin ? rr : rhi) * p.d) * p.n;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                bv[tn][j] = (rin && nok[tn]) ? bp[cn[tn]] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                acc[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv[tn][j], acc[tn], 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int il = i0 + (r / 4) * 8 + hk * 4 + (r % 4);
        if (il >= rows)
            continue;
        float *cp = p.C + ((size_t)b * p.m + rho + (size_t)il * p.d) * p.n;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            if (nok[tn])
                cp[cn[tn]] = acc[tn][r];
    }
}

int check_band(const float *A, const float *B, float *C, int bs, int m, int x, int w, int d,
               const char *what) {
    if (!A || !B || !C)
        return set_error(PET_HIP_ERR_INVALID, "%s: null operand", what);
    if (bs <= 0 || m <= 0 || x <= 0 || w < 0 || d <= 0)
        return set_error(PET_HIP_ERR_INVALID, "%s: bad shape bs=%d m=%d %d w=%d d=%d", what, bs, m,
                         x, w, d);
    const long long band = 2ll * w + 1;
    if ((long long)bs * m * band >= (1ll << 31) || (long long)bs * m * x >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "%s: tensors of 2^31 elements or more", what);
    if ((long long)bs * d > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "%s: batch * dilation = %lld", what,
                         (long long)bs * d);
    return PET_HIP_OK;
}

} // namespace

extern "C" {

int pet_hip_g2bmm_f32(const float *A, const float *B, float *C, int bs, int m, int k, int width,
                      int dilation, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (int rc = check_band(A, B, C, bs, m, k, width, dilation, "g2bmm"))
        return rc;
    BandParams p{A, B, C, bs, m, k, width, dilation, 0, 0, 0};
    p.mc = (m + dilation - 1) / dilation;
    // tiles from column i0 - w to i0 + 31 + w
    p.rtiles = (2 * width + 32 + 31) / 32;
    const unsigned iblocks = (unsigned)((p.mc + 31) / 32);
    if (iblocks > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "g2bmm: %d rows", m);
    dim3 grid((unsigned)p.rtiles, iblocks, (unsigned)(bs * dilation));
    hipLaunchKernelGGL(g2bmm_kernel, grid, dim3(64), 0, as_stream(stream), p);
    return check_launch("g2bmm_kernel");
}

int pet_hip_gbmml_f32(const float *A, const float *B, float *C, int bs, int m, int width, int n,
                      int dilation, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (int rc = check_band(A, B, C, bs, m, n, width, dilation, "gbmml"))
        return rc;
    BandParams p{A, B, C, bs, m, 0, width, dilation, n, 0, 0};
    p.mc = (m + dilation - 1) / dilation;
    const unsigned iblocks = (unsigned)((p.mc + 31) / 32);
    if (iblocks > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "gbmml: %d rows", m);
    if (n > 32) {
        dim3 grid((unsigned)((n + 63) / 64), iblocks, (unsigned)(bs * dilation));
        hipLaunchKernelGGL((gbmml_kernel<2>), grid, dim3(64), 0, as_stream(stream), p);
    } else {
        dim3 grid(1, iblocks, (unsigned)(bs * dilation));
        hipLaunchKernelGGL((gbmml_kernel<1>), grid, dim3(64), 0, as_stream(stream), p);
    }
    return check_launch("gbmml_kernel");
}

} // extern "C"
