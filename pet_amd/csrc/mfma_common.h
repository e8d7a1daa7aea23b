// Shared pieces of the fp32 MFMA contraction kernels: tile shapes, division by
// run-time invariants, the LDS->MFMA inner block and the operand loaders.
#pragma once
#include "common.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace pet {
namespace mfma {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Division by a run-time invariant, branch-free: q = (mulhi(n, mul) + (n & add)) >> shift.
// For d == 1 the multiply contributes nothing and `add` passes n through.
struct FastDiv {
    unsigned d, mul, shift, add;
};

inline FastDiv make_fastdiv(unsigned d) {
    FastDiv f;
    f.d = d;
    f.mul = 0;
    f.shift = 0;
    f.add = 0xFFFFFFFFu;
    if (d <= 1)
        return f;
    f.add = 0;
    unsigned l = 0;
    while ((1ull << l) < d)
        ++l;
    unsigned p = 31 + l;
    f.mul = (unsigned)(((1ull << p) + d - 1) / d);
    f.shift = p - 32;
    return f;
}

__device__ __forceinline__ unsigned fd_div(unsigned n, const FastDiv &f) {
    return (__umulhi(n, f.mul) + (n & f.add)) >> f.shift;
}

template <int BM_, int BN_, int BK_, int WGM_, int WGN_>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_;
    static constexpr int WGM = WGM_, WGN = WGN_;
    static constexpr int NW = WGM * WGN;
    static constexpr int NT = NW * 64;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int KH = BK / 2;
    static constexpr int A_LD = BK + 4;
    static constexpr int B_LD = BN + 4;
    static constexpr int A_ELEMS = BM * A_LD;
    static constexpr int B_ELEMS = BK * B_LD;
    static constexpr int STAGE = A_ELEMS + B_ELEMS;
    // loader shapes
    static constexpr int A_VPT = BM * BK / 4 / NT; // float4 per thread, k-contiguous A
    static constexpr int B_VPT = BK * BN / 4 / NT; // float4 per thread, n-contiguous B
    static constexpr int RPW = BK / NW;            // gather rows per wave (conv)
    static constexpr int PPL = BN / 64;            // gather pixels per lane (conv)
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BK % 8 == 0, "BK must be a multiple of 8");
    static_assert(A_VPT >= 1 && B_VPT >= 1 && RPW >= 1 && PPL >= 1, "tile too small");
    static_assert(BM * BK / 4 % NT == 0 && BK * BN / 4 % NT == 0 && BK % NW == 0 &&
                      BN % 64 == 0,
                  "loader shapes must divide evenly");
};

// ---- the MFMA inner product over one BK block ---------------------------------
template <class Cfg>
__device__ __forceinline__ void mma_block(const float *__restrict__ As,
                                          const float *__restrict__ Bs,
                                          floatx16 (&acc)[Cfg::TM][Cfg::TN], int wm0, int wn0,
                                          int lane) {
    const int l32 = lane & 31, hk = lane >> 5;
    float a[Cfg::TM][Cfg::KH];
#pragma unroll
    for (int tm = 0; tm < Cfg::TM; ++tm) {
        const float *ap = As + (wm0 + tm * 32 + l32) * Cfg::A_LD + hk * Cfg::KH;
#pragma unroll
        for (int j = 0; j < Cfg::KH; j += 4) {
            float4 v = *reinterpret_cast<const float4 *>(ap + j);
            a[tm][j] = v.x;
            a[tm][j + 1] = v.y;
            a[tm][j + 2] = v.z;
            a[tm][j + 3] = v.w;
        }
    }
#pragma unroll
    for (int j = 0; j < Cfg::KH; ++j) {
        float b[Cfg::TN];
        const float *bp = Bs + (hk * Cfg::KH + j) * Cfg::B_LD + wn0 + l32;
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn)
            b[tn] = bp[tn * 32];
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < Cfg::TN; ++tn)
                acc[tm][tn] =
                    __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][j], b[tn], acc[tm][tn], 0, 0, 0);
    }
}

// Sixteen bytes of zeros: a load that must yield 0 (a padding tap, the K tail)
// is pointed here instead of being masked after the fact, so that no
// instruction depends on the loaded value until it is written to LDS.
__device__ __attribute__((aligned(16))) const float g_zero16[4] = {0.f, 0.f, 0.f, 0.f};

// ---- operand loaders -----------------------------------------------------------
// "KC": the operand is stored with K contiguous (weights [f][k], A [m][k],
// B^T [n][k]); "XC": the non-K index is contiguous (A^T [k][m], B [k][n]).
// rows = extent of the non-K index, ld = source row stride.

// K-contiguous source -> registers, branch-free: rows past the end re-read the
// last row (those accumulator rows are never stored), the K tail is zeroed by a
// select. VEC: ld % 4 == 0, K % 4 == 0 and a 16-byte aligned base.
template <int ROWS, int BK, int NT, bool VEC>
__device__ __forceinline__ void load_kc(const float *__restrict__ src, unsigned ld, int row0,
                                        int rows, int k0, int K, int tid,
                                        float4 (&regs)[ROWS * BK / 4 / NT]) {
    constexpr int VPT = ROWS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int row = v / (BK / 4), kq = (v % (BK / 4)) * 4;
        int gr = min(row0 + row, rows - 1), gk = k0 + kq;
        const unsigned rbase = (unsigned)gr * ld;
        float4 val;
        const float *pz = g_zero16;
        if (VEC) {
            const float *q = gk < K ? src + (rbase + (unsigned)gk) : pz;
            val = *reinterpret_cast<const float4 *>(q);
        } else {
            val.x = *(gk < K ? src + (rbase + (unsigned)gk) : pz);
            val.y = *(gk + 1 < K ? src + (rbase + (unsigned)gk + 1u) : pz);
            val.z = *(gk + 2 < K ? src + (rbase + (unsigned)gk + 2u) : pz);
            val.w = *(gk + 3 < K ? src + (rbase + (unsigned)gk + 3u) : pz);
        }
        regs[i] = val;
    }
}

// registers (from load_kc) -> LDS laid out [row][k] with stride LD (used for A)
template <int ROWS, int BK, int NT, int LD>
__device__ __forceinline__ void store_kc_rowmajor(float *__restrict__ dst, int tid,
                                                  const float4 (&regs)[ROWS * BK / 4 / NT]) {
    constexpr int VPT = ROWS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int row = v / (BK / 4), kq = (v % (BK / 4)) * 4;
        *reinterpret_cast<float4 *>(dst + row * LD + kq) = regs[i];
    }
}

// registers (from load_kc) -> LDS laid out [k][row] with stride LD (used for B^T)
template <int ROWS, int BK, int NT, int LD>
__device__ __forceinline__ void store_kc_transposed(float *__restrict__ dst, int tid,
                                                    const float4 (&regs)[ROWS * BK / 4 / NT]) {
    constexpr int VPT = ROWS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int row = v / (BK / 4), kq = (v % (BK / 4)) * 4;
        dst[(kq + 0) * LD + row] = regs[i].x;
        dst[(kq + 1) * LD + row] = regs[i].y;
        dst[(kq + 2) * LD + row] = regs[i].z;
        dst[(kq + 3) * LD + row] = regs[i].w;
    }
}

// X-contiguous source (element (x, k) at src[k * ld + x]) -> registers,
// branch-free in the same way (columns past the end are never stored).
template <int COLS, int BK, int NT, bool VEC>
__device__ __forceinline__ void load_xc(const float *__restrict__ src, unsigned ld, int col0,
                                        int cols, int k0, int K, int tid,
                                        float4 (&regs)[COLS * BK / 4 / NT]) {
    constexpr int VPT = COLS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int k = v / (COLS / 4), cq = (v % (COLS / 4)) * 4;
        int gk = k0 + k, gc = col0 + cq;
        const unsigned kbase = (unsigned)min(gk, K - 1) * ld;
        const float *pz = g_zero16;
        const bool kok = gk < K;
        float4 val;
        if (VEC) {
            const float *q = kok ? src + (kbase + (unsigned)min(gc, cols - 4)) : pz;
            val = *reinterpret_cast<const float4 *>(q);
        } else {
            val.x = *(kok ? src + (kbase + (unsigned)min(gc, cols - 1)) : pz);
            val.y = *(kok ? src + (kbase + (unsigned)min(gc + 1, cols - 1)) : pz);
            val.z = *(kok ? src + (kbase + (unsigned)min(gc + 2, cols - 1)) : pz);
            val.w = *(kok ? src + (kbase + (unsigned)min(gc + 3, cols - 1)) : pz);
        }
        regs[i] = val;
    }
}

// registers (from load_xc) -> LDS [k][col] with stride LD (used for B)
template <int COLS, int BK, int NT, int LD>
__device__ __forceinline__ void store_xc_rowmajor(float *__restrict__ dst, int tid,
                                                  const float4 (&regs)[COLS * BK / 4 / NT]) {
    constexpr int VPT = COLS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int k = v / (COLS / 4), cq = (v % (COLS / 4)) * 4;
        *reinterpret_cast<float4 *>(dst + k * LD + cq) = regs[i];
    }
}

// registers (from load_xc) -> LDS [col][k] with stride LD (used for A^T)
template <int COLS, int BK, int NT, int LD>
__device__ __forceinline__ void store_xc_transposed(float *__restrict__ dst, int tid,
                                                    const float4 (&regs)[COLS * BK / 4 / NT]) {
    constexpr int VPT = COLS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int k = v / (COLS / 4), cq = (v % (COLS / 4)) * 4;
        dst[(cq + 0) * LD + k] = regs[i].x;
        dst[(cq + 1) * LD + k] = regs[i].y;
        dst[(cq + 2) * LD + k] = regs[i].z;
        dst[(cq + 3) * LD + k] = regs[i].w;
    }
}


inline long long tiles_for(int m, int n, int bm, int bn, int batch) {
    return (long long)((m + bm - 1) / bm) * ((n + bn - 1) / bn) * batch;
}

// Tuning knob: PET_HIP_TILE=<n> forces a tile shape (read once).
inline int forced_tile() {
    static int v = [] {
        const char *e = getenv("PET_HIP_TILE");
        return e ? atoi(e) : -1;
    }();
    return v;
}

// conv.hip: non-transposed batched matmul through the plane convolution kernel.
int bmm_as_grouped_1x1(const float *A, const float *B, float *C, const float *bias,
                       const float *res, int b, int m, int n, int k, int act, hipStream_t stream,
                       unsigned flags = 0, int *dry = nullptr);

} // namespace mfma
} // namespace pet
