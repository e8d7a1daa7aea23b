// fp32 MFMA implicit-GEMM convolution for gfx950 (2-D and 3-D, strided, dilated,
// grouped, fused bias + activation). M = output channels of a group, N = output
// pixels (batch folded in), K = (channels per group) x (filter taps).
//
// Two kernels:
//  * conv_plane_kernel: the fast path for 3x3 / 1x1 (and 3x3x3, one kt slice per
//    K step) filters; see the comment at the kernel.
//  * conv_pipe_kernel: any filter shape, stride, dilation and channel count.
// Both keep A (weights) in LDS as [m][k] and B (the im2col tile) as [k][n] and
// feed v_mfma_f32_32x32x2_f32; within a K block MFMA step j gives lanes 0-31
// k = j and lanes 32-63 k = BK/2 + j on both operands.
#include "conv_params.h"

using namespace pet;
using namespace pet::mfma;

namespace {

// ---- convolution -----------------------------------------------------------------



template <class Cfg, bool VECA, bool IS3D>
__global__ __launch_bounds__(Cfg::NT) void conv_pipe_kernel(ConvParams p) {
    __shared__ __attribute__((aligned(16))) float lds[2 * Cfg::STAGE];
    constexpr int KH = Cfg::KH, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int BK = Cfg::BK, NT = Cfg::NT, NW = Cfg::NW;
    constexpr int A_VPT = Cfg::A_VPT, RPW = Cfg::RPW, PPL = Cfg::PPL;
    constexpr int A_LD = Cfg::A_LD, B_LD = Cfg::B_LD;
    constexpr int NM = KH * TM * TN;       // MFMAs (slots) per iteration
    constexpr int NG = A_VPT + RPW;        // prefetch pieces
    constexpr int NWP = NG;                // LDS-write pieces
    constexpr int NRA = TM * (KH / 4);     // A fragment pieces (128-bit reads)
    constexpr int NR = NRA + KH;           // fragment pieces
    constexpr int NP = NG + NWP + 1 + NR;  // + the barrier

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM;
    const int wn0 = (wave % Cfg::WGN) * Cfg::WN;
    const int l32 = lane & 31, hk = lane >> 5;
    const int g = blockIdx.z;
    const int m0 = blockIdx.y * Cfg::BM;
    const int n0 = blockIdx.x * Cfg::BN;

    const int THW = p.T * p.H * p.W, HW = p.H * p.W;
    const float *__restrict__ wg_w = p.w + (long long)g * p.M * p.K;
    const float *__restrict__ wg_x = p.x + (long long)g * p.cpg * THW;

    int pbase[PPL], it0[PPL], ih0[PPL], iw0[PPL];
#pragma unroll
    for (int pp = 0; pp < PPL; ++pp) {
        int pix = min(n0 + lane + pp * 64, p.NPIX - 1);
        unsigned n = fd_div(pix, p.fd_opix);
        unsigned rem = pix - n * p.OPIX;
        unsigned ot = 0;
        if (IS3D) {
            ot = fd_div(rem, p.fd_ohw);
            rem -= ot * (p.OH * p.OW);
        }
        unsigned oh = fd_div(rem, p.fd_ow);
        unsigned ow = rem - oh * p.OW;
        it0[pp] = IS3D ? (int)ot * p.st - p.pt : 0;
        ih0[pp] = (int)oh * p.sh - p.ph;
        iw0[pp] = (int)ow * p.sw - p.pw;
        pbase[pp] = (int)n * p.C * THW + it0[pp] * HW + ih0[pp] * p.W + iw0[pp];
    }
    // fixed A-load coordinates of this thread
    unsigned a_rbase[A_VPT];
    int a_kq[A_VPT], a_lds[A_VPT];
#pragma unroll
    for (int i = 0; i < A_VPT; ++i) {
        int v = tid + i * NT;
        int row = v / (BK / 4);
        a_kq[i] = (v % (BK / 4)) * 4;
        a_rbase[i] = (unsigned)min(m0 + row, p.M - 1) * (unsigned)p.K;
        a_lds[i] = row * A_LD + a_kq[i];
    }
    const int a_frag = (wm0 + l32) * A_LD + hk * KH;         // + tm*32*A_LD + j
    const int b_frag = hk * KH * B_LD + wn0 + l32;            // + j*B_LD + tn*32
    const int b_lds = wave * B_LD + lane;                     // + NW*i*B_LD + pp*64

    float4 preA[2][A_VPT];
    float preB[2][RPW][PPL];
    float fa[2][TM][KH];
    float fb[2][KH][TN];
    floatx16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] = 0.f;

    // ---- the pieces; `i` and `set` are constants once the callers are unrolled
    auto g_piece = [&](int set, int i, int k0) __attribute__((always_inline)) {
        if (i < A_VPT) {
            const int gk = k0 + a_kq[i];
            float4 val;
            const float *pz = g_zero16;
            if (VECA) {
                const float *q = gk < p.K ? wg_w + (a_rbase[i] + (unsigned)gk) : pz;
                val = *reinterpret_cast<const float4 *>(q);
            } else {
                val.x = *(gk < p.K ? wg_w + (a_rbase[i] + (unsigned)gk) : pz);
                val.y = *(gk + 1 < p.K ? wg_w + (a_rbase[i] + (unsigned)gk + 1u) : pz);
                val.z = *(gk + 2 < p.K ? wg_w + (a_rbase[i] + (unsigned)gk + 2u) : pz);
                val.w = *(gk + 3 < p.K ? wg_w + (a_rbase[i] + (unsigned)gk + 3u) : pz);
            }
            preA[set][i] = val;
        } else {
            const int row = i - A_VPT;
            const int k = k0 + wave + NW * row; // wave-uniform: scalar unit
            const unsigned c = fd_div(k, p.fd_krs);
            unsigned rem = k - c * p.fd_krs.d;
            unsigned q = 0;
            if (IS3D) {
                q = fd_div(rem, p.fd_rs);
                rem -= q * p.fd_rs.d;
            }
            const unsigned r = fd_div(rem, p.fd_s);
            const unsigned s = rem - r * p.fd_s.d;
            const int qt = (int)q * p.dt, rh = (int)r * p.dh, sw_ = (int)s * p.dw;
            const int koff = (int)c * THW + qt * HW + rh * p.W + sw_;
            const bool kok = k < p.K;
#pragma unroll
            for (int pp = 0; pp < PPL; ++pp) {
                bool ok = kok & ((unsigned)(ih0[pp] + rh) < (unsigned)p.H) &
                          ((unsigned)(iw0[pp] + sw_) < (unsigned)p.W);
                if (IS3D)
                    ok = ok & ((unsigned)(it0[pp] + qt) < (unsigned)p.T);
                const float *q = ok ? wg_x + (unsigned)(pbase[pp] + koff) : g_zero16;
                preB[set][row][pp] = *q;
            }
        }
    };
    auto w_piece = [&](int set, int i, float *st) __attribute__((always_inline)) {
        if (i < A_VPT) {
            *reinterpret_cast<float4 *>(st + a_lds[i]) = preA[set][i];
        } else {
            const int row = i - A_VPT;
#pragma unroll
            for (int pp = 0; pp < PPL; ++pp)
                st[Cfg::A_ELEMS + b_lds + NW * row * B_LD + pp * 64] =
                    p.x_relu ? fmaxf(preB[set][row][pp], 0.f) : preB[set][row][pp];
        }
    };
    auto r_piece = [&](int set, int i, const float *st) __attribute__((always_inline)) {
        if (i < NRA) {
            const int tm = i / (KH / 4), jq = (i % (KH / 4)) * 4;
            float4 v = *reinterpret_cast<const float4 *>(st + a_frag + tm * 32 * A_LD + jq);
            fa[set][tm][jq] = v.x;
            fa[set][tm][jq + 1] = v.y;
            fa[set][tm][jq + 2] = v.z;
            fa[set][tm][jq + 3] = v.w;
        } else {
            const int j = i - NRA;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                fb[set][j][tn] = st[Cfg::A_ELEMS + b_frag + j * B_LD + tn * 32];
        }
    };
    auto wg_barrier = [&]() __attribute__((always_inline)) {
        // LDS writes done, then the workgroup barrier; global prefetches stay in flight
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    const int nk = (p.K + BK - 1) / BK;

    // ---- prologue: tiles 0 and 1 into the prefetch sets, tile 0 into LDS and fragments
#pragma unroll
    for (int i = 0; i < NG; ++i)
        g_piece(0, i, 0);
#pragma unroll
    for (int i = 0; i < NG; ++i)
        g_piece(1, i, BK);
#pragma unroll
    for (int i = 0; i < NWP; ++i)
        w_piece(0, i, lds);
    wg_barrier();
#pragma unroll
    for (int i = 0; i < NR; ++i)
        r_piece(0, i, lds);

    // one iteration: PAR = kt & 1 selects the register sets
    auto iteration = [&](auto parc, int kt) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
        float *nxt = lds + (PAR ^ 1) * Cfg::STAGE;
        const int kpre = (kt + 2) * BK;
#pragma unroll
        for (int s = 0; s < NM; ++s) {
            const int j = s / (TM * TN), tm = (s / TN) % TM, tn = s % TN;
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[PAR][tm][j], fb[PAR][j][tn],
                                                               acc[tm][tn], 0, 0, 0);
            const int pb = (s * NP + NM - 1) / NM, pe = ((s + 1) * NP + NM - 1) / NM;
#pragma unroll
            for (int q = pb; q < pe; ++q) {
                if (q < NG)
                    g_piece(PAR, q, kpre);
                else if (q < NG + NWP)
                    w_piece(PAR ^ 1, q - NG, nxt);
                else if (q == NG + NWP)
                    wg_barrier();
                else
                    r_piece(PAR ^ 1, q - NG - NWP - 1, nxt);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        iteration(std::integral_constant<int, 0>{}, kt);
        iteration(std::integral_constant<int, 1>{}, kt + 1);
    }
    if (kt < nk)
        iteration(std::integral_constant<int, 0>{}, kt);

    // epilogue: bias + activation, NC(T)HW store
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        int pix = n0 + wn0 + tn * 32 + l32;
        if (pix >= p.NPIX)
            continue;
        unsigned n = fd_div(pix, p.fd_opix);
        unsigned rem = pix - n * p.OPIX;
        const long long ybase = ((long long)n * p.F + (long long)g * p.M) * p.OPIX + rem;
        float *__restrict__ yb = p.y + ybase;
        const float *rb = p.res ? p.res + ybase : nullptr;
        const float *__restrict__ bias = p.bias ? p.bias + g * p.M : nullptr;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int f = m0 + wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4);
                if (f < p.M) {
                    float v = acc[tm][tn][r];
                    if (bias)
                        v += bias[f];
                    if (rb) {
                        const float rv = rb[(unsigned)f * (unsigned)p.OPIX];
                        v += p.res_relu ? fmaxf(rv, 0.f) : rv;
                    }
                    yb[(unsigned)f * (unsigned)p.OPIX] = apply_act(v, p.act);
                }
            }
        }
    }
}

// ---- "plane" convolution kernel ----------------------------------------------------
// The fast path for filters whose (r, s) plane is small (3x3, 1x1, also 3x3x3
// taken one kt slice at a time). One K step covers CB input channels times the
// whole RS = r*s plane, so the tap of a B-tile row, its offset inside the image
// and whether it falls into the padding are the same in every step: they are
// worked out once per thread. The loads are raw buffer loads whose voffset is
// that fixed byte offset, or 2^31 for a padding tap, which the buffer range
// check answers with 0; the step only moves the scalar base. Per element and
// step the wave issues one load and half a ds_write and no address arithmetic,
// which is what lets one or two waves per SIMD keep the MFMA pipe busy: a wave
// issues at most one instruction every four cycles, so with one wave per SIMD the
// whole step has to fit in 16 instructions per MFMA.
//
// Schedule of step kt (NM slots, one MFMA each): first half, W(kt+1): prefetch
// registers -> LDS, each piece followed by G(kt+2): global -> the registers just
// emptied; barrier; second half, R(kt+1): LDS -> the other fragment register set.
template <int BM_, int BN_, int WGM_, int WGN_, int RS_, int CB_>
struct PlaneCfg {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_, RS = RS_, CB = CB_;
    static constexpr int BK = RS * CB;
    static constexpr int NW = WGM * WGN, NT = NW * 64;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int KH = BK / 2;
    static constexpr int A_LD = BK + 4, B_LD = BN + 4;
    static constexpr int A_ELEMS = BM * A_LD, B_ELEMS = BK * B_LD;
    static constexpr int STAGE = A_ELEMS + B_ELEMS;
    static constexpr int RPW = BK / NW, PPL = BN / 64;
    static constexpr int A_V4 = BM * BK / 4;              // float4 per A tile (2-D)
    static constexpr int A_VPT = (A_V4 + NT - 1) / NT;
    static constexpr int A_SPT = BM * BK / NT;            // scalars per thread (3-D)
    static_assert(WM % 32 == 0 && WN % 32 == 0 && KH % 4 == 0 && BK % NW == 0 && BN % 64 == 0 &&
                      (BM * BK) % NT == 0,
                  "bad plane tile");
};


// DIM 2: 2-D. DIM 3: 3-D with kt > 1 (one kt slice of a filter row is runs of r*s
// floats, loaded one float at a time). DIM 4: 3-D with kt == 1 (filter rows are
// contiguous as in 2-D and load as 16-byte words). DIM 5: 3-D with kt > 1 and
// filters repacked kt-major, [kt][f][c/g][r][s]: every kt slice is a 2-D filter
// bank and loads as 16-byte words.
template <class Cfg, int DIM, bool SK>
__global__ __launch_bounds__(Cfg::NT) void conv_plane_kernel(ConvParams p) {
    constexpr bool IS3D = DIM != 2;
    constexpr bool SCALAR_A = DIM == 3;
    constexpr bool PACKED = DIM == 5;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int KH = Cfg::KH, TM = Cfg::TM, TN = Cfg::TN, RS = Cfg::RS, CB = Cfg::CB;
    constexpr int BK = Cfg::BK, NT = Cfg::NT, NW = Cfg::NW;
    constexpr int RPW = Cfg::RPW, PPL = Cfg::PPL;
    constexpr int A_LD = Cfg::A_LD, B_LD = Cfg::B_LD;
    constexpr int NA = SCALAR_A ? Cfg::A_SPT : Cfg::A_VPT; // A pieces per thread
    constexpr int NM = KH * TM * TN;                   // slots per step
    constexpr int HALF = NM / 2;
    constexpr int NWP = NA + RPW;                      // W pieces (first half)
    constexpr int NRA = TM * (KH / 4);
    constexpr int NR = NRA + KH;                       // R pieces
    constexpr int NG = NA + RPW;                       // G pieces

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / Cfg::WGN) * Cfg::WM;
    const int wn0 = (wave % Cfg::WGN) * Cfg::WN;
    const int l32 = lane & 31, hk = lane >> 5;
    // stream-K: this workgroup's share of the tiles * nit K steps
    unsigned seg_u = 0, seg_end = 0;
    if (SK) {
        seg_u = fd_div(blockIdx.x * (unsigned)p.sk_units, p.fd_sk_wgs);
        seg_end = fd_div((blockIdx.x + 1) * (unsigned)p.sk_units, p.fd_sk_wgs);
        if (seg_u >= seg_end)
            return;
    }
    for (bool first_seg = true;; first_seg = false) { // one pass unless stream-K
    if (SK && !first_seg)
        __syncthreads(); // the previous segment's LDS reads are over
    const int ncb = p.cpg / CB;
    const int nit_all = ncb * p.KT;
    int g = 0, ks = 0, it_begin, it_end;
    unsigned bx, by;
    if (SK) {
        const unsigned t = fd_div(seg_u, p.fd_sk_nit); // tile; M tiles vary fastest
        it_begin = (int)(seg_u - t * nit_all);
        it_end = min(nit_all, it_begin + (int)(seg_end - seg_u));
        bx = fd_div(t, p.fd_sk_tm);
        by = t - bx * p.sk_tiles_m;
    } else {
    g = fd_div(blockIdx.z, p.fd_splitk);
    ks = blockIdx.z - g * p.splitk; // which share of the K steps
    // ks * nit_all stays far below 2^31 (at most 64 splits)
    it_begin = (int)fd_div((unsigned)(ks * nit_all), p.fd_splitk);
    it_end = (int)fd_div((unsigned)((ks + 1) * nit_all), p.fd_splitk);
    // Workgroups are handed to the 8 XCDs round-robin in launch order, and each
    // XCD has its own L2. Renumber so that an XCD owns one compact band of tiles
    // (xcd_mg M tiles wide) instead of every eighth tile: its L2 then holds
    // 1/8th of the operands rather than all the filters.
    bx = blockIdx.x, by = blockIdx.y;
    if (p.xcd_chunk) {
        const unsigned L = bx + gridDim.x * by;
        const unsigned Lp = (L & 7) * p.xcd_chunk + (L >> 3);
        const unsigned mg = p.xcd_mg;
        const unsigned band = fd_div(Lp, p.fd_band);
        const unsigned in_band = Lp - band * mg * gridDim.x;
        bx = fd_div(in_band, p.fd_mg);
        by = band * mg + (in_band - bx * mg);
    }
    }
    const int m0 = by * Cfg::BM;
    const int n0 = bx * Cfg::BN;

    const int THW = p.T * p.H * p.W, HW = p.H * p.W;
    const int KRS = p.KT * RS; // weights per (f, c)
    // bases: the pad offset is folded into the image base so every voffset is >= 0
    // strides of a channel, a row and a column of x (a view brings its own; 2-D only)
    const int xsc = p.xv.on ? (int)p.xv.sc : THW;
    const int xsh = p.xv.on ? (int)p.xv.sh : p.W;
    const int xsw = p.xv.on ? (int)p.xv.sw : 1;
    const int padoff = p.pt * HW + p.ph * xsh + p.pw * xsw;
    const float *xg = p.x + (long long)g * p.cpg * xsc - padoff;
    // floats per filter row as stored: all of K, or one kt slice of it when packed
    const int a_row = PACKED ? p.cpg * RS : p.K;
    const float *wg = p.w + (long long)g * p.M * a_row;

    // ---- per-thread invariants of the B gather
    unsigned voffB[RPW][PPL];
    int it0[PPL];
    {
        int oh_[PPL], ow_[PPL];
        unsigned pb[PPL];
#pragma unroll
        for (int pp = 0; pp < PPL; ++pp) {
            int pix = min(n0 + lane + pp * 64, p.NPIX - 1);
            unsigned n = fd_div(pix, p.fd_opix);
            unsigned rem = pix - n * p.OPIX;
            unsigned ot = 0;
            if (IS3D) {
                ot = fd_div(rem, p.fd_ohw);
                rem -= ot * (p.OH * p.OW);
            }
            unsigned oh = fd_div(rem, p.fd_ow);
            unsigned ow = rem - oh * p.OW;
            it0[pp] = (int)ot * p.st - p.pt;
            oh_[pp] = (int)oh * p.sh;
            ow_[pp] = (int)ow * p.sw;
            pb[pp] = (p.xv.on ? view_batch_offset(p.xv, n) : n * (unsigned)(p.C * THW)) +
                     ot * (unsigned)(p.st * HW) + oh_[pp] * xsh + ow_[pp] * xsw;
        }
        // Row i of wave w is row kl = w + NW * i of the B tile, i.e. channel kl / RS and
        // tap kl % RS: the four waves fetch neighbouring taps of one channel at the
        // same time, which the L1 likes. The padding tests depend on the tap only, and
        // with the wave number as a compile-time constant (one copy of this block per
        // wave) so do the tap and all of a row's offsets.
        constexpr int SW = RS == 9 ? 3 : 1; // the host admits 3x3 and 1x1 planes only
        constexpr int SR = RS / SW;
        bool okr[PPL][SR], okc[PPL][SW];
#pragma unroll
        for (int pp = 0; pp < PPL; ++pp) {
#pragma unroll
            for (int r = 0; r < SR; ++r)
                okr[pp][r] = (unsigned)(oh_[pp] + r * p.dh - p.ph) < (unsigned)p.H;
#pragma unroll
            for (int s = 0; s < SW; ++s)
                okc[pp][s] = (unsigned)(ow_[pp] + s * p.dw - p.pw) < (unsigned)p.W;
        }
        auto rows_of = [&](auto wc) __attribute__((always_inline)) {
            constexpr int WV = decltype(wc)::value;
#pragma unroll
            for (int i = 0; i < RPW; ++i) {
                const int kl = WV + NW * i;
                const int cl = kl / RS, t = kl % RS;
                const int r = t / SW, s = t % SW;
                const unsigned roff = (unsigned)(cl * xsc + r * p.dh * xsh + s * p.dw * xsw);
#pragma unroll
                for (int pp = 0; pp < PPL; ++pp)
                    voffB[i][pp] = (okr[pp][r] & okc[pp][s]) ? (pb[pp] + roff) * 4u : kOob;
            }
        };
        static_assert(NW == 2 || NW == 4, "one copy of the row table per wave");
        if (wave == 0)
            rows_of(std::integral_constant<int, 0>{});
        else if (wave == 1)
            rows_of(std::integral_constant<int, 1>{});
        else if (wave == 2)
            rows_of(std::integral_constant<int, 2 % NW>{});
        else
            rows_of(std::integral_constant<int, 3 % NW>{});
    }
    // ---- per-thread invariants of the A loads
    unsigned voffA[NA];
    int ldsA[NA];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        if (SCALAR_A) {
            const int e = tid + i * NT;
            const int f = e / BK, kl = e % BK;
            const int cl = kl / RS, t = kl % RS;
            voffA[i] = ((unsigned)min(m0 + f, p.M - 1) * (unsigned)p.K + cl * KRS + t) * 4u;
            ldsA[i] = f * A_LD + kl;
        } else {
            const int v = tid + i * NT;
            const int row = v / (BK / 4), kq = (v % (BK / 4)) * 4;
            voffA[i] = v < Cfg::A_V4
                           ? ((unsigned)min(m0 + row, p.M - 1) * (unsigned)a_row + kq) * 4u
                           : kOob;
            ldsA[i] = min(row, Cfg::BM - 1) * A_LD + kq;
        }
    }
    const int a_frag = (wm0 + l32) * A_LD + hk * KH;
    const int b_frag = Cfg::A_ELEMS + hk * KH * B_LD + wn0 + l32;
    const int b_lds = Cfg::A_ELEMS + wave * B_LD + lane;

    float4 preA4[SCALAR_A ? 1 : NA];
    float preA1[SCALAR_A ? NA : 1];
    float preB[RPW][PPL];
    float fa[2][TM][KH];
    float fb[2][KH][TN];
    floatx16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] = 0.f;

    // step counters of the prefetch stream: channel block and kt slice
    const int nit = it_end - it_begin;
    int pcb = it_begin / p.KT, pq = it_begin - pcb * p.KT;
    auto advance_prefetch = [&]() __attribute__((always_inline)) {
        // stays on the last step once the end is reached (harmless re-load)
        if (pcb * p.KT + pq + 1 < it_end) {
            if (++pq == p.KT) {
                pq = 0;
                ++pcb;
            }
        }
    };

    // ---- pieces ---------------------------------------------------------------
    auto g_piece = [&](int i) __attribute__((always_inline)) {
        if (i < NA) {
            const unsigned so = PACKED ? (unsigned)(pq * (p.F * a_row) + pcb * CB * RS) * 4u
                                       : (unsigned)(pcb * CB * KRS + pq * RS) * 4u;
            const __amdgpu_buffer_rsrc_t ra = make_rsrc(wg);
            if (SCALAR_A) {
                preA1[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ra, voffA[i], so, 0));
            } else {
                uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(ra, voffA[i], so, 0);
                preA4[i] = make_float4(__uint_as_float(v.x), __uint_as_float(v.y),
                                       __uint_as_float(v.z), __uint_as_float(v.w));
            }
        } else {
            const int row = i - NA;
            const unsigned so = (unsigned)(pcb * CB * xsc + pq * p.dt * HW) * 4u;
            const __amdgpu_buffer_rsrc_t rb = make_rsrc(xg);
#pragma unroll
            for (int pp = 0; pp < PPL; ++pp) {
                unsigned vo = voffB[row][pp];
                if (IS3D)
                    vo = (unsigned)(it0[pp] + pq * p.dt) < (unsigned)p.T ? vo : kOob;
                preB[row][pp] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rb, vo, so, 0));
            }
        }
    };
    auto w_piece = [&](int i, float *st) __attribute__((always_inline)) {
        if (i < NA) {
            if (SCALAR_A) {
                st[ldsA[i]] = preA1[i];
            } else {
                // the last, partly filled round only exists for the first threads
                if ((i + 1) * NT <= Cfg::A_V4 || tid + i * NT < Cfg::A_V4)
                    *reinterpret_cast<float4 *>(st + ldsA[i]) = preA4[i];
            }
        } else {
            const int row = i - NA;
#pragma unroll
            for (int pp = 0; pp < PPL; ++pp)
                st[b_lds + NW * row * B_LD + pp * 64] =
                    p.x_relu ? fmaxf(preB[row][pp], 0.f) : preB[row][pp];
        }
    };
    auto r_piece = [&](int set, int i, const float *st) __attribute__((always_inline)) {
        if (i < NRA) {
            const int tm = i / (KH / 4), jq = (i % (KH / 4)) * 4;
            float4 v = *reinterpret_cast<const float4 *>(st + a_frag + tm * 32 * A_LD + jq);
            fa[set][tm][jq] = v.x;
            fa[set][tm][jq + 1] = v.y;
            fa[set][tm][jq + 2] = v.z;
            fa[set][tm][jq + 3] = v.w;
        } else {
            const int j = i - NRA;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                fb[set][j][tn] = st[b_frag + j * B_LD + tn * 32];
        }
    };
    auto wg_barrier = [&]() __attribute__((always_inline)) {
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    // ---- prologue: step 0 into LDS and fragment set 0, step 1 into the prefetch registers
#pragma unroll
    for (int i = 0; i < NG; ++i)
        g_piece(i);
    advance_prefetch();
#pragma unroll
    for (int i = 0; i < NWP; ++i)
        w_piece(i, lds);
    wg_barrier();
#pragma unroll
    for (int i = 0; i < NR; ++i)
        r_piece(0, i, lds);
#pragma unroll
    for (int i = 0; i < NG; ++i)
        g_piece(i);
    advance_prefetch();

    auto step = [&](auto parc) __attribute__((always_inline)) {
        constexpr int PAR = decltype(parc)::value;
        float *nxt = lds + (PAR ^ 1) * Cfg::STAGE;
#pragma unroll
        for (int s = 0; s < NM; ++s) {
            const int j = s / (TM * TN), tm = (s / TN) % TM, tn = s % TN;
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[PAR][tm][j], fb[PAR][j][tn],
                                                               acc[tm][tn], 0, 0, 0);
            if (s < HALF) {
                // W(kt+1) piece i, then G(kt+2) piece i straight into the registers it
                // has just emptied: a load has a whole step to land
                constexpr int NP = 2 * NWP;
                const int pb_ = (s * NP + HALF - 1) / HALF, pe_ = ((s + 1) * NP + HALF - 1) / HALF;
#pragma unroll
                for (int q = pb_; q < pe_; ++q) {
                    if (q & 1)
                        g_piece(q >> 1);
                    else
                        w_piece(q >> 1, nxt);
                }
                if (s == HALF - 1)
                    wg_barrier();
            } else {
                const int h = s - HALF, HN = NM - HALF;
                const int pb_ = (h * NR + HN - 1) / HN, pe_ = ((h + 1) * NR + HN - 1) / HN;
#pragma unroll
                for (int q = pb_; q < pe_; ++q)
                    r_piece(PAR ^ 1, q, nxt);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        advance_prefetch();
    };
    // Two-level sum: every kFlush steps the running tile is added into a second one and
    // restarted, so no chain of fp32 additions is longer than kFlush * BK + nit / kFlush
    // terms. On a 4608-term contraction (512 channels x 3x3) one chain's rounding error,
    // which grows with the square root of its length, was 1.2e-4 of the smallest outputs
    // against an fp64-accumulated result; 32 vector adds per kFlush steps buy a factor 3.
    constexpr int kFlush = 8;
    floatx16 acc2[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc2[tm][tn][r] = 0.f;
    int kt = 0;
    for (; kt + 1 < nit; kt += 2) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        if (((kt + 2) & (kFlush - 1)) == 0) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        acc2[tm][tn][r] += acc[tm][tn][r];
                        acc[tm][tn][r] = 0.f;
                    }
        }
    }
    if (kt < nit)
        step(std::integral_constant<int, 0>{});
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] += acc2[tm][tn][r];

    // split-K: park the partial tile, and let the workgroup that arrives last add
    // the S partials in a fixed order (the result does not depend on timing).
    // Partials travel as device-scope relaxed atomic stores and loads, which go
    // through to the level where all XCDs agree; the wait below keeps them ahead
    // of the arrival count. Full device fences would also write back and
    // invalidate everything else the L2s hold, which costs tens of microseconds.
    if (p.splitk > 1 && p.sk_mode == 0) {
        const int S = p.splitk;
        const unsigned tile_id = (g * gridDim.y + by) * gridDim.x + bx;
        constexpr int NREG = TM * TN * 16;
        float *mine = p.ws + ((size_t)tile_id * S + ks) * NREG * NT + tid;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(mine + ((tm * TN + tn) * 16 + r) * NT, acc[tm][tn][r],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this lane's partials have landed
        __syncthreads();                                 // ... and every lane's
        int *flag = reinterpret_cast<int *>(lds);
        if (tid == 0)
            *flag = __hip_atomic_fetch_add(&p.cnt[tile_id], 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT) == S - 1;
        __syncthreads();
        if (!*flag)
            return;
        const float *all = p.ws + (size_t)tile_id * S * NREG * NT + tid;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[tm][tn][r] = 0.f;
        // four partial tiles in flight at a time, added in split order
        for (int s2 = 0; s2 < S; s2 += 4) {
            float part[4][NREG];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int r = 0; r < NREG; ++r)
                    part[i][r] = s2 + i < S
                                     ? __hip_atomic_load(all + ((size_t)(s2 + i) * NREG + r) * NT,
                                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                     : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[tm][tn][r] += part[i][(tm * TN + tn) * 16 + r];
        }
        if (tid == 0)
            __hip_atomic_store(&p.cnt[tile_id], 0, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT); // ready for the next launch
    }

    const bool atomic = p.atomic_out;
    if (!atomic && p.vec_out) {
        // epilogue through LDS: the tile is parked as [f][pixel] and leaves as 16-byte
        // words, 256 or 512 contiguous bytes per filter row (the pixel count of an
        // image is a multiple of 4 here, so a word never straddles two images)
        constexpr int C_LD = Cfg::BN + 4;
        constexpr int QPR = Cfg::BN / 4;   // words per tile row
        constexpr int RPP = NT / QPR;      // tile rows per pass
        __syncthreads();                   // every wave is done with the K loop's LDS
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    lds[(wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4)) * C_LD + wn0 + tn * 32 +
                        l32] = acc[tm][tn][r];
        __syncthreads();
        const int q = tid % QPR, r0 = tid / QPR;
        const int pix = n0 + 4 * q;
        if (pix < p.NPIX) {
            const unsigned n = fd_div(pix, p.fd_opix);
            const unsigned rem = pix - n * p.OPIX;
            const long long ybase = ((long long)n * p.F + (long long)g * p.M) * p.OPIX + rem;
            float *__restrict__ yb = p.y + ybase;
            const float *rb = p.res ? p.res + ybase : nullptr;
            const float *__restrict__ bias =
                (p.bias && p.bias_mode == 1) ? p.bias + g * p.M : nullptr;
            float cb[4] = {0.f, 0.f, 0.f, 0.f};
            if (p.bias && p.bias_mode == 2) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    cb[j] = p.bias[rem + j];
            }
#pragma unroll
            for (int pass = 0; pass < Cfg::BM / RPP; ++pass) {
                const int fl = r0 + pass * RPP;
                const int f = m0 + fl;
                if (f < p.M) {
                    float4 v = *reinterpret_cast<const float4 *>(lds + fl * C_LD + 4 * q);
                    const float bf = bias ? bias[f] : 0.f;
                    if (rb) {
                        float4 rv =
                            *reinterpret_cast<const float4 *>(rb + (unsigned)f * (unsigned)p.OPIX);
                        if (p.res_relu)
                            rv = make_float4(fmaxf(rv.x, 0.f), fmaxf(rv.y, 0.f), fmaxf(rv.z, 0.f),
                                             fmaxf(rv.w, 0.f));
                        v.x += rv.x;
                        v.y += rv.y;
                        v.z += rv.z;
                        v.w += rv.w;
                    }
                    v.x = apply_act(v.x + bf + cb[0], p.act);
                    v.y = apply_act(v.y + bf + cb[1], p.act);
                    v.z = apply_act(v.z + bf + cb[2], p.act);
                    v.w = apply_act(v.w + bf + cb[3], p.act);
                    *reinterpret_cast<float4 *>(yb + (unsigned)f * (unsigned)p.OPIX) = v;
                }
            }
        }
        return;
    }

    // epilogue: bias + activation (or the atomic add of a split), NC(T)HW store
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        int pix = n0 + wn0 + tn * 32 + l32;
        if (pix >= p.NPIX)
            continue;
        unsigned n = fd_div(pix, p.fd_opix);
        unsigned rem = pix - n * p.OPIX;
        // floats between two filters' outputs for this pixel, and where the first one goes
        unsigned ysc = (unsigned)p.OPIX;
        long long ybase = ((long long)n * p.F + (long long)g * p.M) * p.OPIX + rem;
        if (p.yv.on) {
            const unsigned oh = fd_div(rem, p.fd_ow);
            ysc = p.yv.sc;
            ybase = (long long)view_batch_offset(p.yv, n) + (long long)g * p.M * ysc +
                    oh * p.yv.sh + (rem - oh * p.OW) * p.yv.sw;
        }
        float *__restrict__ yb = p.y + ybase;
        const float *rb = p.res ? p.res + ybase : nullptr;
        const float *__restrict__ bias =
            (p.bias && p.bias_mode == 1) ? p.bias + g * p.M : nullptr;
        const float colbias = (p.bias && p.bias_mode == 2) ? p.bias[rem] : 0.f;
        if (atomic) {
            // the output was initialised with the bias by a launch before this one;
            // the activation runs in a launch after it
            const bool add_res = p.res_first && it_begin == 0;
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int f = m0 + wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4);
                    if (f < p.M) {
                        float v = acc[tm][tn][r];
                        if (add_res) {
                            const float rv = rb[(unsigned)f * ysc];
                            v += p.res_relu ? fmaxf(rv, 0.f) : rv;
                        }
                        unsafeAtomicAdd(yb + (unsigned)f * ysc, v);
                    }
                }
        } else {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    int f = m0 + wm0 + tm * 32 + (r / 4) * 8 + hk * 4 + (r % 4);
                    if (f < p.M) {
                        float v = acc[tm][tn][r];
                        if (bias)
                            v += bias[f];
                        if (rb) {
                            const float rv = rb[(unsigned)f * ysc];
                            v += p.res_relu ? fmaxf(rv, 0.f) : rv;
                        }
                        yb[(unsigned)f * ysc] = apply_act(v + colbias, p.act);
                    }
                }
        }
    }
    if (!SK)
        break;
    seg_u += it_end - it_begin;
    if (seg_u >= seg_end)
        break;
    } // segments
}

using Cfg128x128 = TileCfg<128, 128, 16, 2, 2>;
using Cfg64x128 = TileCfg<64, 128, 32, 2, 2>;
using Cfg64x64 = TileCfg<64, 64, 32, 2, 2>;
using Cfg32x64 = TileCfg<32, 64, 16, 1, 2>;

template <class Cfg>
int launch_pipe_cfg(const ConvParams &p, bool veca, hipStream_t stream) {
    dim3 grid((p.NPIX + Cfg::BN - 1) / Cfg::BN, (p.M + Cfg::BM - 1) / Cfg::BM, p.G);
    const bool is3d = p.T > 1 || p.KT > 1 || p.pt > 0 || p.st > 1;
    if (is3d) {
        if (veca)
            hipLaunchKernelGGL((conv_pipe_kernel<Cfg, true, true>), grid, dim3(Cfg::NT), 0, stream,
                               p);
        else
            hipLaunchKernelGGL((conv_pipe_kernel<Cfg, false, true>), grid, dim3(Cfg::NT), 0,
                               stream, p);
    } else {
        if (veca)
            hipLaunchKernelGGL((conv_pipe_kernel<Cfg, true, false>), grid, dim3(Cfg::NT), 0,
                               stream, p);
        else
            hipLaunchKernelGGL((conv_pipe_kernel<Cfg, false, false>), grid, dim3(Cfg::NT), 0,
                               stream, p);
    }
    return check_launch("conv_pipe_kernel");
}

// Tile choice of the general kernel: the largest tile that still gives every
// CU a workgroup. 0: 128x128, 1: 64x128, 2: 64x64, 3: 32x64.
int pick_tile(int M, int N, int batch) {
    if (forced_tile() >= 0)
        return forced_tile() & 3;
    const long long want = 256;
    if (M >= 128 && tiles_for(M, N, 128, 128, batch) >= 2 * want)
        return 0;
    if (M >= 64 && tiles_for(M, N, 64, 128, batch) >= want)
        return 1;
    if (M > 32)
        return 2;
    return 3;
}

// Output initialisation for split-K launches: y = bias (per channel or per
// column) or 0, plus the residual if there is one (which may be y itself); the
// partial sums are then added atomically.
__global__ __launch_bounds__(256) void splitk_init_kernel(float *y, const float *__restrict__ bias,
                                                          const float *res, int res_relu,
                                                          int bias_mode, unsigned F, unsigned OPIX,
                                                          size_t total) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t step = (size_t)gridDim.x * 256;
    for (; i < total; i += step) {
        float v = 0.f;
        if (bias) {
            unsigned pix = (unsigned)(i % OPIX);
            unsigned f = (unsigned)((i / OPIX) % F);
            v = bias_mode == 2 ? bias[pix] : bias[f];
        }
        if (res)
            v += res_relu ? fmaxf(res[i], 0.f) : res[i];
        y[i] = v;
    }
}

// Stream-K is instantiated for the 3x3 tiles of 64 rows only (it needs its own copy of the
// kernel: the segment loop's bookkeeping would otherwise push scalars of every launch
// out of the SGPR file).
template <class Cfg>
constexpr bool has_streamk = Cfg::BM >= 64 && Cfg::RS == 9;

// Split-K scratch of pet_hip_conv2d_static_f32, the entry point that allocates nothing:
// partial tiles, then one arrival counter per output tile. Every GPU the library runs on
// holds its own copy until the process ends. In host code the array's name is not a device
// address: static_scratch() asks the runtime for this device's copy once and host code
// uses that pointer everywhere (kernel arguments included).
constexpr size_t kStaticWsElems = (size_t)2 << 20; // 8 MiB of partial tiles
constexpr int kStaticCounters = 4096;
static __device__ __align__(256) float g_static_scratch[kStaticWsElems + kStaticCounters];

constexpr int kMaxDevices = 64;
static float *g_static_ptr[kMaxDevices] = {nullptr};

// Device address of the current device's copy of the array (nullptr + error text on failure).
float *static_scratch() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error(PET_HIP_ERR_RUNTIME, "no current device for the static scratch");
        return nullptr;
    }
    if (!g_static_ptr[dev]) {
        void *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch));
        if (e != hipSuccess || !ptr) {
            set_error(PET_HIP_ERR_RUNTIME, "hipGetSymbolAddress(static scratch) failed: %s",
                      hipGetErrorString(e));
            return nullptr;
        }
        // zero at load; every launch returns its counters to zero before it ends
        g_static_ptr[dev] = static_cast<float *>(ptr);
    }
    return g_static_ptr[dev];
}

template <class Cfg, int DIM>
int launch_plane_cfg(ConvParams p, hipStream_t stream) {
    const size_t lds_bytes = 2 * (size_t)Cfg::STAGE * sizeof(float);
    static int attr_status = [&] {
        hipError_t e = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&conv_plane_kernel<Cfg, DIM, false>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if constexpr (has_streamk<Cfg>) {
            if (e == hipSuccess)
                e = hipFuncSetAttribute(
                    reinterpret_cast<const void *>(&conv_plane_kernel<Cfg, DIM, true>),
                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        }
        return e == hipSuccess ? 0 : 1;
    }();
    if (attr_status)
        return -1; // caller falls back to the general kernel
    const long long tiles = tiles_for(p.M, p.NPIX, Cfg::BM, Cfg::BN, p.G);
    const int nit = (p.cpg / Cfg::CB) * p.KT;
    // Split K when the tiles alone leave CUs idle. A small cost model, in K steps of
    // this tile: the busiest CU runs ceil(tiles * S / 256) workgroups one after the
    // other (co-resident workgroups share its MFMA pipes), each of nit / S steps
    // plus a fixed prologue + epilogue; a split launch pays two more small launches
    // and its atomics contend S ways. Every workgroup keeps at least two steps.
    int splitk = 1;
    const double scale = (double)(Cfg::BM * Cfg::BN) / (64.0 * 64.0);
    const double c_fixed = 3.0 / scale, c_launches = 4.0 / scale, c_contend = 0.1 / scale;
    // A workgroup that has its CU to itself (one wave per SIMD) has nothing to hide its LDS
    // and barrier waits behind: its steps cost about an eighth more than those of two
    // co-resident workgroups, whose prologues and epilogues also overlap. (Measured by the
    // host layer's algorithm search: 256 tiles of 64 steps run faster as 512 workgroups of 32.)
    static const double solo = getenv("PET_HIP_SOLO_COST") ? atof(getenv("PET_HIP_SOLO_COST")) : 1.12;
    // ... on long K loops; short ones are bound by their launches either way
    static const int solo_steps = getenv("PET_HIP_SOLO_STEPS") ? atoi(getenv("PET_HIP_SOLO_STEPS")) : 12;
    const long long r1 = (tiles + 255) / 256;
    const bool legacy = solo <= 0.0; // the model before the occupancy terms (for comparison)
    double best = legacy ? r1 * (nit + c_fixed)
                         : r1 * nit * (r1 == 1 && nit >= solo_steps ? solo : 1.0) +
                               ((r1 + 1) / 2) * c_fixed; // S = 1
    if ((legacy ? tiles < 256 : tiles <= 256) && nit >= 4) {
        static const int max_env =
            getenv("PET_HIP_SPLITK_MAX") ? atoi(getenv("PET_HIP_SPLITK_MAX")) : 64;
        for (int S = 1; S <= std::min(nit / 2, max_env); ++S) {
            const long long rounds = (tiles * S + 255) / 256;
            double cost = legacy ? rounds * ((nit + S - 1) / S + c_fixed)
                                 : rounds * ((nit + S - 1) / S) *
                                           (rounds == 1 && (nit + S - 1) / S >= solo_steps ? solo
                                                                                           : 1.0) +
                                       ((rounds + 1) / 2) * c_fixed;
            if (S > 1)
                cost += c_launches + c_contend * S;
            if (S == 1 || cost < best) {
                best = cost;
                splitk = S;
            }
        }
    }
    static const int forced_env = getenv("PET_HIP_SPLITK") ? atoi(getenv("PET_HIP_SPLITK")) : 0;
    const int forced = p.force_splitk > 0 ? p.force_splitk : forced_env;
    if (forced > 0)
        splitk = std::min(forced, nit);
    if ((long long)p.G * splitk > 65535)
        splitk = 1;
    // Stream-K instead: 256 (64x128 tiles) or 512 workgroups share the tiles * nit K
    // steps evenly, so no CU waits for a last, partly filled round of tiles. All
    // sums go into y as float atomics (initialising launch before, activation after).
    // Taken when the model sees 5 % less work on the busiest CU (its workgroups also sit two
    // to a CU where a short grid of tiles leaves one: measured, a margin of 10 % left the
    // 128->128 and 256->256 3x3x3 layers of R3D-18 on split K, 18 % and 9 % slower; at
    // no margin the 512->512 layers of the dilated block turn 3 % slower).
    p.streamk = 0;
    {
        static const int sk_env0 = getenv("PET_HIP_STREAMK") ? atoi(getenv("PET_HIP_STREAMK")) : -1;
        const int sk_env = p.force_streamk >= 0 ? p.force_streamk : sk_env0;
        const long long units = tiles * nit;
        const int wgs = Cfg::BM * Cfg::BN >= 64 * 128 ? 256 : 512;
        const double cost_sk = (double)units / 256 + 2 * c_fixed + c_launches;
        static const double sk_margin =
            getenv("PET_HIP_STREAMK_MARGIN") ? atof(getenv("PET_HIP_STREAMK_MARGIN")) : 0.95;
        const bool fits = p.G == 1 && units * (wgs + 1) < (1ll << 31) && units >= 2 * wgs &&
                          has_streamk<Cfg> && !deterministic() && !p.static_ws;
        if (fits && forced <= 0 && (sk_env == 1 || (sk_env != 0 && cost_sk < sk_margin * best))) {
            p.streamk = 1;
            splitk = 1;
            p.sk_units = (int)units;
            p.sk_tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM;
            p.fd_sk_wgs = make_fastdiv((unsigned)wgs);
            p.fd_sk_nit = make_fastdiv((unsigned)nit);
            p.fd_sk_tm = make_fastdiv((unsigned)p.sk_tiles_m);
        }
    }
    // Float atomics into the output (an initialising launch before, the activation
    // in a launch after) are the faster way by 10-30% on small layers: the ordered
    // single-launch sum adds three dependent round trips through memory to every
    // tile. It is used when bit-reproducible results are asked for.
    p.sk_mode = (deterministic() || p.static_ws) ? 0 : 1;
    if (splitk > 1 && p.sk_mode == 0 && p.static_ws) {
        // the static array of this file; a shape that does not fit is refused, not shrunk
        const size_t need = (size_t)tiles * Cfg::BM * Cfg::BN * splitk;
        if (need > kStaticWsElems || tiles > kStaticCounters)
            return set_error(PET_HIP_ERR_UNSUPPORTED,
                             "this convolution splits K %d ways over %lld tiles and needs %zu "
                             "bytes of scratch; the static scratch holds %zu bytes and %d tiles",
                             splitk, tiles, need * sizeof(float),
                             kStaticWsElems * sizeof(float), kStaticCounters);
        if (!p.dry_atomic) {
            float *base = static_scratch();
            if (!base)
                return PET_HIP_ERR_RUNTIME;
            p.ws = base;
            p.cnt = reinterpret_cast<int *>(base + kStaticWsElems);
        }
    } else if (splitk > 1 && p.sk_mode == 0) {
        // the partial tiles and arrival counters live in the library's scratch
        size_t ws_elems;
        int ncnt;
        splitk_workspace(&p.ws, &ws_elems, &p.cnt, &ncnt);
        const size_t per_split = (size_t)tiles * Cfg::BM * Cfg::BN;
        while (splitk > 1 && per_split * splitk > ws_elems)
            splitk /= 2;
        if (tiles > ncnt || splitk < 2)
            splitk = 1;
    }
    p.splitk = splitk;
    p.atomic_out = p.streamk || (splitk > 1 && p.sk_mode == 1);
    dim3 grid((p.NPIX + Cfg::BN - 1) / Cfg::BN, (p.M + Cfg::BM - 1) / Cfg::BM, p.G * splitk);
    // XCD bands: only when every z plane starts on XCD 0 and has several tiles per XCD
    p.xcd_chunk = 0;
    p.xcd_mg = 1;
    static const bool xcd_off = getenv("PET_HIP_XCD") && atoi(getenv("PET_HIP_XCD")) == 0;
    const unsigned plane_tiles = grid.x * grid.y;
    if (!xcd_off && !p.streamk && plane_tiles % 8 == 0 && plane_tiles >= 64) {
        const unsigned chunk = plane_tiles / 8;
        // bytes an XCD pulls for a band mg tiles wide: its filters + its pixels
        double best = 0;
        for (unsigned mg = 1; mg <= grid.y; mg *= 2) {
            if (grid.y % mg || chunk % mg)
                continue;
            const double cost = (double)mg * Cfg::BM * p.K +
                                (double)(chunk / mg) * Cfg::BN * p.cpg * p.st * p.sh * p.sw;
            if (best == 0 || cost < best) {
                best = cost;
                p.xcd_mg = (int)mg;
            }
        }
        p.xcd_chunk = (int)chunk;
    }
    if (p.dry_atomic) {
        *p.dry_atomic = p.atomic_out;
        return PET_HIP_OK;
    }
    p.res_first = p.atomic_out && p.y_init && p.res != nullptr;
    if (p.atomic_out && !p.y_init) {
        int rc = launch_accumulate_init(p, stream);
        if (rc)
            return rc;
    }
    p.fd_splitk = make_fastdiv((unsigned)p.splitk);
    p.fd_mg = make_fastdiv((unsigned)p.xcd_mg);
    p.fd_band = make_fastdiv((unsigned)p.xcd_mg * grid.x);
    p.vec_out = (p.OPIX % 4 == 0) && (((uintptr_t)p.y & 15) == 0) &&
                (((uintptr_t)p.res & 15) == 0) && !p.yv.on;
    if constexpr (has_streamk<Cfg>) {
        if (p.streamk) {
            grid = dim3(Cfg::BM * Cfg::BN >= 64 * 128 ? 256 : 512, 1, 1);
            hipLaunchKernelGGL((conv_plane_kernel<Cfg, DIM, true>), grid, dim3(Cfg::NT), lds_bytes,
                               stream, p);
        }
    }
    if (!p.streamk)
        hipLaunchKernelGGL((conv_plane_kernel<Cfg, DIM, false>), grid, dim3(Cfg::NT), lds_bytes,
                           stream, p);
    int rc = check_launch("conv_plane_kernel");
    if (rc == PET_HIP_OK && p.atomic_out && p.act != PET_HIP_ACT_NONE &&
        !(p.defer_relu && p.act == PET_HIP_ACT_RELU))
        rc = pet_hip_activation(p.y, p.y, (size_t)p.NPIX * p.F, p.act, (pet_hip_stream_t)stream);
    return rc;
}

template <int RS, int CB>
int launch_plane(const ConvParams &p, bool is3d, hipStream_t stream) {
    using C64x128 = PlaneCfg<64, 128, 2, 2, RS, CB>;
    using C64x64 = PlaneCfg<64, 64, 2, 2, RS, CB>;
    using C32x64 = PlaneCfg<32, 64, 1, 2, RS, CB>;
    // 64x64 tiles, two workgroups to a CU (each hides the other's prologue, epilogue and
    // barrier waits), measured equal or better than one 64x128 workgroup per CU up to
    // a few rounds of tiles; beyond that 64x128 wins through its lower LDS traffic per
    // MFMA (2048 tiles of 64x128 with 8 steps: 212 vs 230 us). 32x64 for M <= 32.
    // The 3-D kernel stays with 64x64: with kt-major filters R3D-18 layer 1 takes 117 us
    // against 121 us with 64x128 tiles.
    int tile = p.M > 32 ? 1 : 2;
    if (p.M > 32 && !is3d && tiles_for(p.M, p.NPIX, 64, 64, p.G) > 2048)
        tile = 0;
    if (forced_tile() >= 0)
        tile = forced_tile() % 3;
    const int dim = !is3d ? 2 : (p.KT == 1 ? 4 : (p.wpacked ? 5 : 3));
    if (tile == 0)
        return dim == 2   ? launch_plane_cfg<C64x128, 2>(p, stream)
               : dim == 3 ? launch_plane_cfg<C64x128, 3>(p, stream)
               : dim == 4 ? launch_plane_cfg<C64x128, 4>(p, stream)
                          : launch_plane_cfg<C64x128, 5>(p, stream);
    if (tile == 1)
        return dim == 2   ? launch_plane_cfg<C64x64, 2>(p, stream)
               : dim == 3 ? launch_plane_cfg<C64x64, 3>(p, stream)
               : dim == 4 ? launch_plane_cfg<C64x64, 4>(p, stream)
                          : launch_plane_cfg<C64x64, 5>(p, stream);
    return dim == 2   ? launch_plane_cfg<C32x64, 2>(p, stream)
           : dim == 3 ? launch_plane_cfg<C32x64, 3>(p, stream)
           : dim == 4 ? launch_plane_cfg<C32x64, 4>(p, stream)
                      : launch_plane_cfg<C32x64, 5>(p, stream);
}

// Returns -1 when the plane kernel does not apply.
int try_launch_plane(const ConvParams &p, hipStream_t stream) {
    static const bool off = getenv("PET_HIP_PLANE") && atoi(getenv("PET_HIP_PLANE")) == 0;
    if (off)
        return -1;
    // voffsets count from the image base minus the pad offset
    const long long in_bytes =
        4ll * p.N * p.C * p.T * p.H * p.W +
        (p.xv.on ? 4ll * ((long long)p.ph * p.xv.sh + (long long)p.pw * p.xv.sw) : 0);
    const long long w_bytes = 4ll * p.F * p.K;
    if (in_bytes >= (1ll << 31) || w_bytes >= (1ll << 31))
        return -1;
    if (((uintptr_t)p.w & 15) != 0 || p.w_shared || p.bias_gstride)
        return -1;
    const bool is3d = p.T > 1 || p.KT > 1 || p.pt > 0 || p.st > 1;
    if (is3d && (p.xv.on || p.yv.on))
        return -1;
    const int rs = p.R * p.S;
    if (rs == 9 && p.R == 3 && p.cpg % 8 == 0)
        return launch_plane<9, 8>(p, is3d, stream);
    if (rs == 1 && p.cpg % 32 == 0)
        return launch_plane<1, 32>(p, is3d, stream);
    return -1;
}

// Shapes whose kt slices the plane kernel reads as 2-D filter banks.
bool packed_filters_apply(long long f, int cpg, int kt, int r, int s) {
    static const bool off = getenv("PET_HIP_PLANE") && atoi(getenv("PET_HIP_PLANE")) == 0;
    if (off || kt <= 1 || 4ll * f * cpg * kt * r * s >= (1ll << 31))
        return false;
    return (r == 3 && s == 3 && cpg % 8 == 0) || (r == 1 && s == 1 && cpg % 32 == 0);
}

__global__ void pack_filters_kernel(const float *__restrict__ w, float *__restrict__ out,
                                    unsigned rows, unsigned kt, unsigned rs) {
    // out[q][row][t] = w[row][q][t], row = f * cpg + c
    const unsigned total = rows * kt * rs;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += gridDim.x * blockDim.x) {
        const unsigned t = i % rs, row = (i / rs) % rows, q = i / (rs * rows);
        out[i] = w[(row * kt + q) * rs + t];
    }
}

int launch_conv(ConvParams &p, hipStream_t stream) {
    int rc = try_launch_direct(p, stream);
    if (rc >= 0)
        return rc;
    rc = try_launch_plane(p, stream);
    if (rc >= 0)
        return rc;
    if (p.xv.on || p.yv.on)
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "strided operands are read by the kernels for 3x3 filters over a "
                         "multiple of 8 channels and 1x1 filters over a multiple of 32 only "
                         "(pet_hip_conv2d_view_supported would have said so)");
    if (p.wpacked)
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "kt-major filters are only read by the plane kernel; this shape does "
                         "not use it (pet_hip_conv3d_pack_filters would have said so)");
    if (p.dry_atomic) // the kernels below never accumulate into y
        return PET_HIP_OK;
    rc = try_launch_stem(p, stream);
    if (rc >= 0)
        return rc;
    const bool veca = (p.K % 4 == 0) && (((uintptr_t)p.w & 15) == 0);
    switch (pick_tile(p.M, p.NPIX, p.G)) {
    case 0:
        return launch_pipe_cfg<Cfg128x128>(p, veca, stream);
    case 1:
        return launch_pipe_cfg<Cfg64x128>(p, veca, stream);
    case 2:
        return launch_pipe_cfg<Cfg64x64>(p, veca, stream);
    default:
        return launch_pipe_cfg<Cfg32x64>(p, veca, stream);
    }
}

// Checks that the strides of a view visit every float of a dense buffer of n * c * h * w
// floats once (sorted by stride, each factor starts where the ones below it end) and
// copies them for the kernels.
bool take_view(const pet_hip_conv_view &v, int n, int c, int h, int w, OperandView &out) {
    const long long e0 = v.n_extent[0], e1 = v.n_extent[1];
    if (e0 < 1 || e1 < 1 || e0 * e1 > n || n % (e0 * e1) != 0)
        return false;
    struct Factor {
        long long ext, stride;
    } fs[6] = {{e0, v.n_stride[0]}, {e1, v.n_stride[1]}, {n / (e0 * e1), v.n_stride[2]},
               {c, v.c_stride},     {h, v.h_stride},     {w, v.w_stride}};
    // factors that are stepped along, by stride; the others go last
    std::sort(fs, fs + 6, [](const Factor &a, const Factor &b) {
        return std::make_pair(a.ext == 1, a.stride) < std::make_pair(b.ext == 1, b.stride);
    });
    long long want = 1;
    for (const Factor &f : fs) {
        if (f.ext == 1)
            continue; // never stepped along: its stride is not looked at
        if (f.stride != want)
            return false;
        want *= f.ext;
    }
    out.on = 1;
    out.sc = (unsigned)v.c_stride;
    out.sh = (unsigned)v.h_stride;
    out.sw = (unsigned)v.w_stride;
    out.fd_ne0 = make_fastdiv((unsigned)e0);
    out.fd_ne1 = make_fastdiv((unsigned)e1);
    for (int i = 0; i < 3; ++i)
        out.ns[i] = (unsigned)v.n_stride[i];
    if (e0 == 1)
        out.ns[0] = 0;
    if (e1 == 1)
        out.ns[1] = 0;
    if (n == e0 * e1)
        out.ns[2] = 0;
    if (c == 1)
        out.sc = 1; // multiplied by channel 0 only; also a divisor in the initialising launch
    if (h == 1)
        out.sh = 0;
    if (w == 1)
        out.sw = 0;
    return true;
}

// Algorithm override (PET_HIP_CONV_ALGO, 0: the cost model decides): forced K shares per
// tile and / or stream-K on or off.
void apply_algo(ConvParams &p, unsigned algo) {
    static const int kSplit[PET_HIP_CONV_ALGO_COUNT] = {0, 1, 2, 4, 8, 16, 0, 0};
    p.force_splitk = algo < PET_HIP_CONV_ALGO_COUNT ? kSplit[algo] : 0;
    p.force_streamk = algo == 0 ? -1 : (algo == 6 ? 1 : 0);
}

int conv_common(const float *x, const float *w, const float *bias, float *y, int n, int c, int t,
                int h, int wd, int f, int kt, int r, int s, int pt, int ph, int pw, int st, int sh,
                int sw, int dt, int dh, int dw, int groups, int act, hipStream_t stream,
                bool wpacked = false, const float *res = nullptr, unsigned flags = 0,
                int *dry = nullptr, bool static_ws = false,
                const pet_hip_conv_view *xview = nullptr,
                const pet_hip_conv_view *yview = nullptr) {
    if (flags & ~(unsigned)(PET_HIP_CALL_Y_INITIALISED | PET_HIP_CALL_DEFER_RELU |
                            PET_HIP_CALL_X_RELU | PET_HIP_CALL_RES_RELU | 0xff00u))
        return set_error(PET_HIP_ERR_INVALID, "unknown call flags 0x%x", flags);
    if ((flags & PET_HIP_CALL_DEFER_RELU) && act != PET_HIP_ACT_RELU)
        return set_error(PET_HIP_ERR_INVALID, "only a ReLU can be left to the readers");
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
    if (dry) {
        // shape query: the operands only have to look aligned
        x = w = reinterpret_cast<const float *>(uintptr_t(256));
        y = reinterpret_cast<float *>(uintptr_t(512));
        *dry = 0;
    }
    if (!x || !w || !y)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    if (res == y)
        return set_error(PET_HIP_ERR_INVALID, "the residual must not be the output buffer");
    p.x = x;
    p.w = w;
    p.bias = bias;
    p.res = res;
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
    p.bias_mode = 1;
    p.splitk = 1;
    p.x_relu = (flags & PET_HIP_CALL_X_RELU) != 0;
    p.res_relu = (flags & PET_HIP_CALL_RES_RELU) != 0;
    p.y_init = (flags & PET_HIP_CALL_Y_INITIALISED) != 0;
    p.defer_relu = (flags & PET_HIP_CALL_DEFER_RELU) != 0;
    p.dry_atomic = dry;
    p.static_ws = static_ws;
    if (xview || yview) {
        if (t != 1 || kt != 1 || pt != 0 || st != 1 || dt != 1)
            return set_error(PET_HIP_ERR_INVALID, "strided operands are for 2-D convolutions");
        if (xview && !take_view(*xview, n, c, h, wd, p.xv))
            return set_error(PET_HIP_ERR_INVALID,
                             "x_view does not address a dense [%d,%d,%d,%d] buffer", n, c, h, wd);
        if (yview && !take_view(*yview, n, f, p.OH, p.OW, p.yv))
            return set_error(PET_HIP_ERR_INVALID,
                             "y_view does not address a dense [%d,%d,%d,%d] buffer", n, f, p.OH,
                             p.OW);
    }
    if (((flags >> 8) & 0xffu) >= PET_HIP_CONV_ALGO_COUNT)
        return set_error(PET_HIP_ERR_INVALID, "unknown convolution algorithm %u",
                         (flags >> 8) & 0xffu);
    apply_algo(p, (flags >> 8) & 0xffu);
    p.wpacked = wpacked;
    if (wpacked && !packed_filters_apply(f, c / groups, kt, r, s))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "no kt-major form for this filter shape");
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

namespace pet {
namespace mfma {

// Batched row-major matmul without transposes is a grouped 1x1 convolution:
// the batch is the group, B[b] ([k][n]) is that group's k-channel "image" of n
// pixels, A[b] ([m][k]) its filters. Returns -1 when the plane kernel does not
// apply (k not a multiple of 32, operands above 2 GiB, misaligned A).
int bmm_as_grouped_1x1(const float *A, const float *B, float *C, const float *bias,
                       const float *res, int b, int m, int n, int k, int act, hipStream_t stream,
                       unsigned flags, int *dry) {
    if (k % 32 != 0 || b > 65535)
        return -1;
    const bool a_shared = (flags & PET_HIP_CALL_A_SHARED) != 0;
    const bool bias_per_batch = (flags & PET_HIP_CALL_BIAS_PER_BATCH) != 0;
    // the group view holds b*k "channels" of n pixels and b*m "filters" of k taps: both
    // must stay inside 32-bit element counts and the 2 GiB range of a buffer resource
    if ((long long)b * k >= (1ll << 31) || (long long)b * m >= (1ll << 31) ||
        4ll * b * k * n >= (1ll << 31) || 4ll * b * m * k >= (1ll << 31) ||
        (long long)b * m * n >= (1ll << 31))
        return -1;
    ConvParams p;
    memset(&p, 0, sizeof(p));
    p.y_init = (flags & PET_HIP_CALL_Y_INITIALISED) != 0;
    p.dry_atomic = dry;
    apply_algo(p, (flags >> 8) & 0xffu);
    p.x = B;
    p.w = A;
    p.bias = bias;
    p.res = res;
    p.y = C;
    p.N = 1;
    p.C = b * k;
    p.T = 1;
    p.H = 1;
    p.W = n;
    p.F = b * m;
    p.KT = p.R = p.S = 1;
    p.st = p.sh = p.sw = p.dt = p.dh = p.dw = 1;
    p.G = b;
    p.cpg = k;
    p.OT = p.OH = 1;
    p.OW = n;
    p.M = m;
    p.K = k;
    p.NPIX = n;
    p.OPIX = n;
    p.act = act;
    p.bias_mode = 2;
    p.splitk = 1;
    p.fd_krs = make_fastdiv(1);
    p.fd_rs = make_fastdiv(1);
    p.fd_s = make_fastdiv(1);
    p.fd_opix = make_fastdiv((unsigned)n);
    p.fd_ohw = make_fastdiv((unsigned)n);
    p.fd_ow = make_fastdiv((unsigned)n);
    p.fd_splitk = make_fastdiv(1);
    p.w_shared = a_shared;
    p.bias_gstride = bias_per_batch ? n : 0;
    const int rc = try_launch_direct(p, stream);
    return rc >= 0 ? rc : try_launch_plane(p, stream);
}

int launch_accumulate_init(const ConvParams &p, hipStream_t stream) {
    const size_t total = (size_t)p.NPIX * p.F;
    unsigned igrid = (unsigned)std::min<size_t>((total + 255) / 256, 4096);
    hipLaunchKernelGGL(splitk_init_kernel, dim3(igrid), dim3(256), 0, stream, p.y, p.bias, p.res,
                       p.res_relu, p.bias_mode, (unsigned)p.F,
                       // floats per channel run: a viewed y is a dense buffer whose channel
                       // factor has this stride
                       p.yv.on ? p.yv.sc : (unsigned)p.OPIX, total);
    return check_launch("splitk_init_kernel");
}

} // namespace mfma
} // namespace pet

extern "C" {

int pet_hip_conv2d_f32(const float *x, const float *w, const float *bias, float *y, int n, int c,
                       int h, int wd, int f, int r, int s, int ph, int pw, int sh, int sw, int dh,
                       int dw, int groups, int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream));
}

int pet_hip_conv2d_static_f32(const float *x, const float *w, const float *bias, float *y, int n,
                              int c, int h, int wd, int f, int r, int s, int ph, int pw, int sh,
                              int sw, int dh, int dw, int groups, int act,
                              pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream), false, nullptr, 0, nullptr, true);
}

int pet_hip_conv3d_f32(const float *x, const float *w, const float *bias, float *y, int n, int c,
                       int t, int h, int wd, int f, int kt, int r, int s, int pt, int ph, int pw,
                       int st, int sh, int sw, int dt, int dh, int dw, int groups, int act,
                       pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, t, h, wd, f, kt, r, s, pt, ph, pw, st, sh, sw, dt, dh,
                       dw, groups, act, as_stream(stream));
}

int pet_hip_conv2d_res_f32(const float *x, const float *w, const float *bias,
                           const float *residual, float *y, int n, int c, int h, int wd, int f,
                           int r, int s, int ph, int pw, int sh, int sw, int dh, int dw, int groups,
                           int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream), false, residual);
}

int pet_hip_conv3d_res_f32(const float *x, const float *w, int w_is_packed, const float *bias,
                           const float *residual, float *y, int n, int c, int t, int h, int wd,
                           int f, int kt, int r, int s, int pt, int ph, int pw, int st, int sh,
                           int sw, int dt, int dh, int dw, int groups, int act,
                           pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, t, h, wd, f, kt, r, s, pt, ph, pw, st, sh, sw, dt, dh,
                       dw, groups, act, as_stream(stream), w_is_packed != 0, residual);
}

int pet_hip_conv2d_ex_f32(const float *x, const float *w, const float *bias,
                          const float *residual, float *y, int n, int c, int h, int wd, int f,
                          int r, int s, int ph, int pw, int sh, int sw, int dh, int dw, int groups,
                          int act, unsigned flags, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream), false, residual, flags);
}

int pet_hip_conv3d_ex_f32(const float *x, const float *w, int w_is_packed, const float *bias,
                          const float *residual, float *y, int n, int c, int t, int h, int wd,
                          int f, int kt, int r, int s, int pt, int ph, int pw, int st, int sh,
                          int sw, int dt, int dh, int dw, int groups, int act, unsigned flags,
                          pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, t, h, wd, f, kt, r, s, pt, ph, pw, st, sh, sw, dt, dh,
                       dw, groups, act, as_stream(stream), w_is_packed != 0, residual, flags);
}

int pet_hip_conv2d_view_f32(const float *x, const pet_hip_conv_view *x_view, const float *w,
                            const float *bias, const float *residual, float *y,
                            const pet_hip_conv_view *y_view, int n, int c, int h, int wd, int f,
                            int r, int s, int ph, int pw, int sh, int sw, int dh, int dw,
                            int groups, int act, unsigned flags, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, w, bias, y, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1, sh, sw, 1, dh, dw,
                       groups, act, as_stream(stream), false, residual, flags, nullptr, false,
                       x_view, y_view);
}

int pet_hip_conv2d_view_supported(int n, int c, int h, int wd, int f, int r, int s, int ph, int pw,
                                  int sh, int sw, int dh, int dw, int groups, int *yes) {
    PET_REQUIRE_INIT();
    if (!yes)
        return set_error(PET_HIP_ERR_INVALID, "null result pointer");
    // the shape with x in its usual layout, said as a view
    pet_hip_conv_view plain;
    plain.w_stride = 1;
    plain.h_stride = wd;
    plain.c_stride = (long long)h * wd;
    plain.n_extent[0] = plain.n_extent[1] = 1;
    plain.n_stride[0] = plain.n_stride[1] = 0;
    plain.n_stride[2] = (long long)c * h * wd;
    int accumulates = 0;
    const int rc = conv_common(nullptr, nullptr, nullptr, nullptr, n, c, 1, h, wd, f, 1, r, s, 0, ph,
                               pw, 1, sh, sw, 1, dh, dw, groups, PET_HIP_ACT_NONE, nullptr, false,
                               nullptr, 0, &accumulates, false, &plain, nullptr);
    *yes = rc == PET_HIP_OK;
    return rc == PET_HIP_ERR_UNSUPPORTED ? PET_HIP_OK : rc;
}

int pet_hip_conv2d_accumulates(int n, int c, int h, int wd, int f, int r, int s, int ph, int pw,
                               int sh, int sw, int dh, int dw, int groups, int *yes) {
    PET_REQUIRE_INIT();
    if (!yes)
        return set_error(PET_HIP_ERR_INVALID, "null result pointer");
    return conv_common(nullptr, nullptr, nullptr, nullptr, n, c, 1, h, wd, f, 1, r, s, 0, ph, pw, 1,
                       sh, sw, 1, dh, dw, groups, PET_HIP_ACT_NONE, nullptr, false, nullptr, 0, yes);
}

int pet_hip_conv3d_accumulates(int n, int c, int t, int h, int wd, int f, int kt, int r, int s,
                               int pt, int ph, int pw, int st, int sh, int sw, int dt, int dh,
                               int dw, int groups, int w_is_packed, int *yes) {
    PET_REQUIRE_INIT();
    if (!yes)
        return set_error(PET_HIP_ERR_INVALID, "null result pointer");
    return conv_common(nullptr, nullptr, nullptr, nullptr, n, c, t, h, wd, f, kt, r, s, pt, ph, pw,
                       st, sh, sw, dt, dh, dw, groups, PET_HIP_ACT_NONE, nullptr, w_is_packed != 0,
                       nullptr, 0, yes);
}

int pet_hip_conv3d_pack_filters(const float *w, float *packed, int f, int cpg, int kt, int r,
                                int s, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (f <= 0 || cpg <= 0 || kt <= 0 || r <= 0 || s <= 0)
        return set_error(PET_HIP_ERR_INVALID, "bad filter shape");
    if (!packed_filters_apply(f, cpg, kt, r, s))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "no kt-major form for this filter shape");
    if (!w || !packed || w == packed)
        return set_error(PET_HIP_ERR_INVALID, "filters and their packed copy must be two buffers");
    const unsigned rows = (unsigned)f * (unsigned)cpg, total = rows * kt * r * s;
    const unsigned blocks = std::min<unsigned>((total + 255) / 256, 4096);
    hipLaunchKernelGGL(pack_filters_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), w,
                       packed, rows, (unsigned)kt, (unsigned)(r * s));
    return check_launch("pack_filters_kernel");
}

int pet_hip_conv3d_packed_f32(const float *x, const float *packed, const float *bias, float *y,
                              int n, int c, int t, int h, int wd, int f, int kt, int r, int s,
                              int pt, int ph, int pw, int st, int sh, int sw, int dt, int dh,
                              int dw, int groups, int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return conv_common(x, packed, bias, y, n, c, t, h, wd, f, kt, r, s, pt, ph, pw, st, sh, sw, dt,
                       dh, dw, groups, act, as_stream(stream), true);
}

} // extern "C"
