// fp32 MFMA contractions for gfx950: implicit-GEMM convolution (2-D and 3-D,
// strided / dilated / grouped, fused bias + activation) and batched matmul.
//
// One tiling serves both. A workgroup of NW waves owns a BM x BN tile of the
// output (M = output channels or matmul rows, N = output pixels or matmul
// columns) and walks K in steps of BK:
//   global -> registers (tile kt+1)   overlapped with
//   LDS -> v_mfma_f32_32x32x2_f32     (tile kt), then registers -> LDS.
// LDS holds A as [m][k] (k contiguous, row stride BK+4 so that a lane's BK/2
// k-values are two 128-bit reads) and B as [k][n] (n contiguous). Within a BK
// block MFMA step j feeds lanes 0-31 with k = j and lanes 32-63 with
// k = BK/2 + j, for both operands, so the products pair up correctly whatever
// the order.
#include "common.h"

#include <algorithm>

using namespace pet;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct FastDiv {
    unsigned d, mul, shift;
};

FastDiv make_fastdiv(unsigned d) {
    FastDiv f;
    f.d = d;
    f.mul = 0;
    f.shift = 0;
    if (d <= 1)
        return f;
    unsigned l = 0;
    while ((1ull << l) < d)
        ++l;
    unsigned p = 31 + l;
    f.mul = (unsigned)(((1ull << p) + d - 1) / d);
    f.shift = p - 32;
    return f;
}

__device__ __forceinline__ unsigned fd_div(unsigned n, const FastDiv &f) {
    return f.d == 1 ? n : (__umulhi(n, f.mul) >> f.shift);
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

// ---- operand loaders -----------------------------------------------------------
// "KC": the operand is stored with K contiguous (weights [f][k], A [m][k],
// B^T [n][k]); "XC": the non-K index is contiguous (A^T [k][m], B [k][n]).
// rows = extent of the non-K index, ld = source row stride.

// K-contiguous source -> registers. VEC: ld % 4 == 0 and 16-byte aligned base.
template <int ROWS, int BK, int NT, bool VEC>
__device__ __forceinline__ void load_kc(const float *__restrict__ src, long long ld, int row0,
                                        int rows, int k0, int K, int tid,
                                        float4 (&regs)[ROWS * BK / 4 / NT]) {
    constexpr int VPT = ROWS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int row = v / (BK / 4), kq = (v % (BK / 4)) * 4;
        int gr = row0 + row, gk = k0 + kq;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (gr < rows) {
            const float *p = src + (long long)gr * ld + gk;
            if (VEC) {
                if (gk < K)
                    val = *reinterpret_cast<const float4 *>(p);
            } else {
                if (gk < K)
                    val.x = p[0];
                if (gk + 1 < K)
                    val.y = p[1];
                if (gk + 2 < K)
                    val.z = p[2];
                if (gk + 3 < K)
                    val.w = p[3];
            }
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

// X-contiguous source (element (x, k) at src[k * ld + x]) -> registers.
template <int COLS, int BK, int NT, bool VEC>
__device__ __forceinline__ void load_xc(const float *__restrict__ src, long long ld, int col0,
                                        int cols, int k0, int K, int tid,
                                        float4 (&regs)[COLS * BK / 4 / NT]) {
    constexpr int VPT = COLS * BK / 4 / NT;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        int v = tid + i * NT;
        int k = v / (COLS / 4), cq = (v % (COLS / 4)) * 4;
        int gk = k0 + k, gc = col0 + cq;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (gk < K) {
            const float *p = src + (long long)gk * ld + gc;
            if (VEC) {
                if (gc < cols)
                    val = *reinterpret_cast<const float4 *>(p);
            } else {
                if (gc < cols)
                    val.x = p[0];
                if (gc + 1 < cols)
                    val.y = p[1];
                if (gc + 2 < cols)
                    val.z = p[2];
                if (gc + 3 < cols)
                    val.w = p[3];
            }
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

// ---- convolution -----------------------------------------------------------------

struct ConvParams {
    const float *x, *w, *bias;
    float *y;
    int N, C, T, H, W, F;
    int KT, R, S;
    int pt, ph, pw, st, sh, sw, dt, dh, dw;
    int G, cpg;
    int OT, OH, OW;
    int M;    // output channels per group
    int K;    // cpg * KT * R * S
    int NPIX; // N * OT * OH * OW
    int OPIX; // OT * OH * OW
    int act;
    FastDiv fd_krs, fd_rs, fd_s;     // k -> (c, kt, r, s)
    FastDiv fd_opix, fd_ohw, fd_ow;  // pixel -> (n, ot, oh, ow)
    int tiles_n;                     // pixel tiles (for the workgroup swizzle)
};

template <class Cfg, bool VECA>
__global__ __launch_bounds__(Cfg::NT) void conv_igemm_kernel(ConvParams p) {
    __shared__ __attribute__((aligned(16))) float lds[2 * Cfg::STAGE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM;
    const int wn0 = (wave % Cfg::WGN) * Cfg::WN;
    const int g = blockIdx.z;
    const int m0 = blockIdx.y * Cfg::BM;
    const int n0 = blockIdx.x * Cfg::BN;

    const int THW = p.T * p.H * p.W, HW = p.H * p.W;
    const float *__restrict__ wg_w = p.w + (long long)g * p.M * p.K;
    const float *__restrict__ wg_x = p.x + (long long)g * p.cpg * THW;

    // per-lane pixel state: PPL pixels, fixed for the whole kernel
    int pbase[Cfg::PPL], it0[Cfg::PPL], ih0[Cfg::PPL], iw0[Cfg::PPL];
#pragma unroll
    for (int pp = 0; pp < Cfg::PPL; ++pp) {
        int pix = n0 + lane + pp * 64;
        if (pix < p.NPIX) {
            unsigned n = fd_div(pix, p.fd_opix);
            unsigned rem = pix - n * p.OPIX;
            unsigned ot = fd_div(rem, p.fd_ohw);
            rem -= ot * (p.OH * p.OW);
            unsigned oh = fd_div(rem, p.fd_ow);
            unsigned ow = rem - oh * p.OW;
            it0[pp] = (int)ot * p.st - p.pt;
            ih0[pp] = (int)oh * p.sh - p.ph;
            iw0[pp] = (int)ow * p.sw - p.pw;
            pbase[pp] = (int)n * p.C * THW + it0[pp] * HW + ih0[pp] * p.W + iw0[pp];
        } else {
            it0[pp] = ih0[pp] = iw0[pp] = -(1 << 28); // never in range
            pbase[pp] = 0;
        }
    }

    float4 areg[Cfg::A_VPT];
    float breg[Cfg::RPW][Cfg::PPL];

    auto gather_b = [&](int k0) {
#pragma unroll
        for (int i = 0; i < Cfg::RPW; ++i) {
            const int k = k0 + wave + Cfg::NW * i; // wave-uniform
            const unsigned c = fd_div(k, p.fd_krs);
            unsigned rem = k - c * p.fd_krs.d;
            const unsigned q = fd_div(rem, p.fd_rs);
            rem -= q * p.fd_rs.d;
            const unsigned r = fd_div(rem, p.fd_s);
            const unsigned s = rem - r * p.fd_s.d;
            const int qt = (int)q * p.dt, rh = (int)r * p.dh, sw_ = (int)s * p.dw;
            const int koff = (int)c * THW + qt * HW + rh * p.W + sw_;
            const bool kok = k < p.K;
#pragma unroll
            for (int pp = 0; pp < Cfg::PPL; ++pp) {
                bool ok = kok && (unsigned)(it0[pp] + qt) < (unsigned)p.T &&
                          (unsigned)(ih0[pp] + rh) < (unsigned)p.H &&
                          (unsigned)(iw0[pp] + sw_) < (unsigned)p.W;
                float v = 0.f;
                if (ok)
                    v = wg_x[pbase[pp] + koff];
                breg[i][pp] = v;
            }
        }
    };
    auto store_b = [&](float *Bs) {
#pragma unroll
        for (int i = 0; i < Cfg::RPW; ++i)
#pragma unroll
            for (int pp = 0; pp < Cfg::PPL; ++pp)
                Bs[(wave + Cfg::NW * i) * Cfg::B_LD + lane + pp * 64] = breg[i][pp];
    };

    floatx16 acc[Cfg::TM][Cfg::TN];
#pragma unroll
    for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] = 0.f;

    const int nk = (p.K + Cfg::BK - 1) / Cfg::BK;
    load_kc<Cfg::BM, Cfg::BK, Cfg::NT, VECA>(wg_w, p.K, m0, p.M, 0, p.K, tid, areg);
    gather_b(0);
    store_kc_rowmajor<Cfg::BM, Cfg::BK, Cfg::NT, Cfg::A_LD>(lds, tid, areg);
    store_b(lds + Cfg::A_ELEMS);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        float *cur = lds + (kt & 1) * Cfg::STAGE;
        float *nxt = lds + ((kt + 1) & 1) * Cfg::STAGE;
        const bool more = kt + 1 < nk;
        if (more) {
            load_kc<Cfg::BM, Cfg::BK, Cfg::NT, VECA>(wg_w, p.K, m0, p.M, (kt + 1) * Cfg::BK, p.K,
                                                     tid, areg);
            gather_b((kt + 1) * Cfg::BK);
        }
        mma_block<Cfg>(cur, cur + Cfg::A_ELEMS, acc, wm0, wn0, lane);
        if (more) {
            store_kc_rowmajor<Cfg::BM, Cfg::BK, Cfg::NT, Cfg::A_LD>(nxt, tid, areg);
            store_b(nxt + Cfg::A_ELEMS);
        }
        __syncthreads();
    }

    // epilogue: bias + activation, NC(T)HW store. Lane holds column l%32 and
    // rows (r/4)*8 + (l/32)*4 + r%4 of each 32x32 block.
    const int l32 = lane & 31, hk = lane >> 5;
#pragma unroll
    for (int tn = 0; tn < Cfg::TN; ++tn) {
        int pix = n0 + wn0 + tn * 32 + l32;
        if (pix >= p.NPIX)
            continue;
        unsigned n = fd_div(pix, p.fd_opix);
        unsigned rem = pix - n * p.OPIX;
        long long obase = ((long long)n * p.F + (long long)g * p.M) * p.OPIX + rem;
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int f = m0 + wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4);
                if (f < p.M) {
                    float v = acc[tm][tn][r];
                    if (p.bias)
                        v += p.bias[g * p.M + f];
                    p.y[obase + (long long)f * p.OPIX] = apply_act(v, p.act);
                }
            }
        }
    }
}

// ---- batched matmul ----------------------------------------------------------------

struct GemmParams {
    const float *A, *B, *bias;
    float *C;
    int M, N, K;
    long long sA, sB, sC; // batch strides
    int act;
};

template <class Cfg, bool TA, bool TB, bool VEC>
__global__ __launch_bounds__(Cfg::NT) void bmm_kernel(GemmParams p) {
    __shared__ __attribute__((aligned(16))) float lds[2 * Cfg::STAGE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM;
    const int wn0 = (wave % Cfg::WGN) * Cfg::WN;
    const int b = blockIdx.z;
    const int m0 = blockIdx.y * Cfg::BM;
    const int n0 = blockIdx.x * Cfg::BN;
    const float *__restrict__ A = p.A + (long long)b * p.sA;
    const float *__restrict__ B = p.B + (long long)b * p.sB;
    float *__restrict__ C = p.C + (long long)b * p.sC;

    float4 areg[Cfg::A_VPT];
    float4 breg[Cfg::B_VPT];

    auto load_tiles = [&](int k0) {
        if (TA)
            load_xc<Cfg::BM, Cfg::BK, Cfg::NT, VEC>(A, p.M, m0, p.M, k0, p.K, tid, areg);
        else
            load_kc<Cfg::BM, Cfg::BK, Cfg::NT, VEC>(A, p.K, m0, p.M, k0, p.K, tid, areg);
        if (TB)
            load_kc<Cfg::BN, Cfg::BK, Cfg::NT, VEC>(B, p.K, n0, p.N, k0, p.K, tid, breg);
        else
            load_xc<Cfg::BN, Cfg::BK, Cfg::NT, VEC>(B, p.N, n0, p.N, k0, p.K, tid, breg);
    };
    auto store_tiles = [&](float *st) {
        if (TA)
            store_xc_transposed<Cfg::BM, Cfg::BK, Cfg::NT, Cfg::A_LD>(st, tid, areg);
        else
            store_kc_rowmajor<Cfg::BM, Cfg::BK, Cfg::NT, Cfg::A_LD>(st, tid, areg);
        if (TB)
            store_kc_transposed<Cfg::BN, Cfg::BK, Cfg::NT, Cfg::B_LD>(st + Cfg::A_ELEMS, tid, breg);
        else
            store_xc_rowmajor<Cfg::BN, Cfg::BK, Cfg::NT, Cfg::B_LD>(st + Cfg::A_ELEMS, tid, breg);
    };

    floatx16 acc[Cfg::TM][Cfg::TN];
#pragma unroll
    for (int tm = 0; tm < Cfg::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < Cfg::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] = 0.f;

    const int nk = (p.K + Cfg::BK - 1) / Cfg::BK;
    load_tiles(0);
    store_tiles(lds);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        float *cur = lds + (kt & 1) * Cfg::STAGE;
        float *nxt = lds + ((kt + 1) & 1) * Cfg::STAGE;
        const bool more = kt + 1 < nk;
        if (more)
            load_tiles((kt + 1) * Cfg::BK);
        mma_block<Cfg>(cur, cur + Cfg::A_ELEMS, acc, wm0, wn0, lane);
        if (more)
            store_tiles(nxt);
        __syncthreads();
    }

    const int l32 = lane & 31, hk = lane >> 5;
#pragma unroll
    for (int tn = 0; tn < Cfg::TN; ++tn) {
        int col = n0 + wn0 + tn * 32 + l32;
        if (col >= p.N)
            continue;
        float bv = p.bias ? p.bias[col] : 0.f;
#pragma unroll
        for (int tm = 0; tm < Cfg::TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int row = m0 + wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4);
                if (row < p.M)
                    C[(long long)row * p.N + col] = apply_act(acc[tm][tn][r] + bv, p.act);
            }
        }
    }
}

// Tile menu. Picked per problem so that the grid fills the 256 CUs.
using Cfg128x128 = TileCfg<128, 128, 16, 2, 2>;
using Cfg64x128 = TileCfg<64, 128, 16, 2, 2>;
using Cfg64x64 = TileCfg<64, 64, 16, 2, 2>;
using Cfg32x64 = TileCfg<32, 64, 16, 1, 2>;

template <class Cfg>
int launch_conv_cfg(const ConvParams &p, bool veca, hipStream_t stream) {
    dim3 grid((p.NPIX + Cfg::BN - 1) / Cfg::BN, (p.M + Cfg::BM - 1) / Cfg::BM, p.G);
    if (veca)
        hipLaunchKernelGGL((conv_igemm_kernel<Cfg, true>), grid, dim3(Cfg::NT), 0, stream, p);
    else
        hipLaunchKernelGGL((conv_igemm_kernel<Cfg, false>), grid, dim3(Cfg::NT), 0, stream, p);
    return check_launch("conv_igemm_kernel");
}

long long tiles_for(int m, int n, int bm, int bn, int batch) {
    return (long long)((m + bm - 1) / bm) * ((n + bn - 1) / bn) * batch;
}

// 0: 128x128, 1: 64x128, 2: 64x64, 3: 32x64
int pick_tile(int M, int N, int batch) {
    const long long want = 256; // one workgroup per CU at least
    if (M >= 128 && tiles_for(M, N, 128, 128, batch) >= 2 * want)
        return 0;
    if (M >= 64 && tiles_for(M, N, 64, 128, batch) >= want)
        return 1;
    if (M >= 64 && tiles_for(M, N, 64, 64, batch) >= want / 2)
        return 2;
    if (M > 32)
        return 2;
    return 3;
}

int launch_conv(ConvParams &p, hipStream_t stream) {
    bool veca = (p.K % 4 == 0) && (((uintptr_t)p.w & 15) == 0);
    switch (pick_tile(p.M, p.NPIX, p.G)) {
    case 0:
        return launch_conv_cfg<Cfg128x128>(p, veca, stream);
    case 1:
        return launch_conv_cfg<Cfg64x128>(p, veca, stream);
    case 2:
        return launch_conv_cfg<Cfg64x64>(p, veca, stream);
    default:
        return launch_conv_cfg<Cfg32x64>(p, veca, stream);
    }
}

template <class Cfg, bool TA, bool TB>
int launch_bmm_cfg(const GemmParams &p, int batch, bool vec, hipStream_t stream) {
    dim3 grid((p.N + Cfg::BN - 1) / Cfg::BN, (p.M + Cfg::BM - 1) / Cfg::BM, batch);
    if (vec)
        hipLaunchKernelGGL((bmm_kernel<Cfg, TA, TB, true>), grid, dim3(Cfg::NT), 0, stream, p);
    else
        hipLaunchKernelGGL((bmm_kernel<Cfg, TA, TB, false>), grid, dim3(Cfg::NT), 0, stream, p);
    return check_launch("bmm_kernel");
}

template <bool TA, bool TB>
int launch_bmm_t(const GemmParams &p, int batch, bool vec, hipStream_t stream) {
    switch (pick_tile(p.M, p.N, batch)) {
    case 0:
        return launch_bmm_cfg<Cfg128x128, TA, TB>(p, batch, vec, stream);
    case 1:
        return launch_bmm_cfg<Cfg64x128, TA, TB>(p, batch, vec, stream);
    case 2:
        return launch_bmm_cfg<Cfg64x64, TA, TB>(p, batch, vec, stream);
    default:
        return launch_bmm_cfg<Cfg32x64, TA, TB>(p, batch, vec, stream);
    }
}

int conv_common(const float *x, const float *w, const float *bias, float *y, int n, int c, int t,
                int h, int wd, int f, int kt, int r, int s, int pt, int ph, int pw, int st, int sh,
                int sw, int dt, int dh, int dw, int groups, int act, hipStream_t stream) {
    if (n < 0 || c <= 0 || t <= 0 || h <= 0 || wd <= 0 || f <= 0 || kt <= 0 || r <= 0 || s <= 0 ||
        groups <= 0 || st <= 0 || sh <= 0 || sw <= 0 || dt <= 0 || dh <= 0 || dw <= 0 || pt < 0 ||
        ph < 0 || pw < 0)
        return set_error(PET_HIP_ERR_INVALID, "bad convolution arguments");
    if (act < PET_HIP_ACT_NONE || act > PET_HIP_ACT_GELU)
        return set_error(PET_HIP_ERR_INVALID, "unknown activation %d", act);
    // ConvOp::compute returns nullptr when f % g != 0; checkValid needs c % cpg == 0
    if (c % groups != 0 || f % groups != 0)
        return set_error(PET_HIP_ERR_INVALID,
                         "channels (%d) and filters (%d) must be divisible by groups (%d)", c, f,
                         groups);
    ConvParams p;
    memset(&p, 0, sizeof(p));
    p.OT = pet_hip_conv_out_dim(t, kt, pt, st, dt);
    p.OH = pet_hip_conv_out_dim(h, r, ph, sh, dh);
    p.OW = pet_hip_conv_out_dim(wd, s, pw, sw, dw);
    if (p.OT < 0 || p.OH < 0 || p.OW < 0)
        return set_error(PET_HIP_ERR_INVALID, "kernel larger than the padded input");
    long long opix = (long long)p.OT * p.OH * p.OW;
    long long npix = opix * n;
    long long in_elems = (long long)n * c * t * h * wd;
    long long out_elems = npix * f;
    long long kk = (long long)(c / groups) * kt * r * s;
    if (npix == 0)
        return PET_HIP_OK; // empty output
    if (in_elems >= (1ll << 31) || out_elems >= (1ll << 31) || kk >= (1ll << 30) ||
        (long long)f * kk >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "convolution operands above 2^31 elements");
    if (!x || !w || !y)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    p.x = x;
    p.w = w;
    p.bias = bias;
    p.y = y;
    p.N = n;
    p.C = c;
    p.T = t;
    p.H = h;
    p.W = wd;
    p.F = f;
    p.KT = kt;
    p.R = r;
    p.S = s;
    p.pt = pt;
    p.ph = ph;
    p.pw = pw;
    p.st = st;
    p.sh = sh;
    p.sw = sw;
    p.dt = dt;
    p.dh = dh;
    p.dw = dw;
    p.G = groups;
    p.cpg = c / groups;
    p.M = f / groups;
    p.K = (int)kk;
    p.NPIX = (int)npix;
    p.OPIX = (int)opix;
    p.act = act;
    p.fd_krs = make_fastdiv((unsigned)(kt * r * s));
    p.fd_rs = make_fastdiv((unsigned)(r * s));
    p.fd_s = make_fastdiv((unsigned)s);
    p.fd_opix = make_fastdiv((unsigned)opix);
    p.fd_ohw = make_fastdiv((unsigned)(p.OH * p.OW));
    p.fd_ow = make_fastdiv((unsigned)p.OW);
    if (groups > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "more than 65535 groups");
    return launch_conv(p, stream);
}

} // namespace

extern "C" {

int pet_hip_conv2d_f32(const float *x, const float *w, const float *bias, float *y, int n, int c,
                       int h, int wd, int f, int r, int s, int ph, int pw, int sh, int sw, int dh,
                       int dw, int groups, int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream));
}

int pet_hip_conv3d_f32(const float *x, const float *w, const float *bias, float *y, int n, int c,
                       int t, int h, int wd, int f, int kt, int r, int s, int pt, int ph, int pw,
                       int st, int sh, int sw, int dt, int dh, int dw, int groups, int act,
                       pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, t, h, wd, f, kt, r, s, pt, ph, pw, st, sh, sw, dt, dh,
                       dw, groups, act, as_stream(stream));
}

int pet_hip_bmm_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                    const float *B, float *C, const float *bias, int act,
                    pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (b < 0 || m < 0 || n < 0 || k < 0)
        return set_error(PET_HIP_ERR_INVALID, "negative matmul dims");
    if (act < PET_HIP_ACT_NONE || act > PET_HIP_ACT_GELU)
        return set_error(PET_HIP_ERR_INVALID, "unknown activation %d", act);
    if ((long long)b * m * n == 0)
        return PET_HIP_OK;
    if (!A || !B || !C)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    if ((long long)m * k >= (1ll << 31) || (long long)k * n >= (1ll << 31) ||
        (long long)m * n >= (1ll << 31) || b > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "matmul operand too large");
    GemmParams p;
    p.A = A;
    p.B = B;
    p.C = C;
    p.bias = bias;
    p.M = m;
    p.N = n;
    p.K = k;
    p.sA = (long long)m * k;
    p.sB = (long long)k * n;
    p.sC = (long long)m * n;
    p.act = act;
    // float4 loads need every row start 16-byte aligned on both operands
    long long lda = transA ? m : k, ldb = transB ? k : n;
    bool vec = lda % 4 == 0 && ldb % 4 == 0 && p.sA % 4 == 0 && p.sB % 4 == 0 &&
               (((uintptr_t)A | (uintptr_t)B) & 15) == 0 &&
               (transA ? m % 4 == 0 : k % 4 == 0) && (transB ? k % 4 == 0 : n % 4 == 0);
    hipStream_t s = as_stream(stream);
    if (transA)
        return transB ? launch_bmm_t<true, true>(p, b, vec, s)
                      : launch_bmm_t<true, false>(p, b, vec, s);
    return transB ? launch_bmm_t<false, true>(p, b, vec, s)
                  : launch_bmm_t<false, false>(p, b, vec, s);
}

} // extern "C"
