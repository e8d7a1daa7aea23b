// Register-fed fp32 MFMA contraction for small problems (batch-1 ResNet / BERT layers):
// 3x3 and 1x1 convolutions, and matmul as a grouped 1x1 convolution.
//
// The LDS-staged kernels of conv.hip need a few hundred 64x64 tiles and a long K loop to
// hide their fixed costs (address tables, first loads, epilogue); a 0.2 GFLOP layer has
// neither. Here a wave owns a (32 TM) x (32 TN) output tile and a share of K, and feeds
// v_mfma_f32_32x32x2_f32 straight from global memory:
//  * A (filters, K contiguous): lane (l32, hk) holds row m0 + l32, k = hk * KH + j for
//    MFMA step j, i.e. a contiguous run of the row. Loaded that way every lane of a load
//    would touch a cache line of its own (rows are K floats apart), which made the L1 the
//    limit of the whole kernel; so a wave reads its 32 x KC tile as consecutive 16-byte
//    words (a row is KC/4 neighbouring lanes), parks it in a private LDS region and reads
//    it back in operand order. No barrier: only the wave itself touches the region.
//  * B (im2col): lane (l32, hk) holds pixel n0 + l32; one K chunk is CB channels times the
//    whole r*s plane, the upper half-wave takes the upper CB/2 channels, so a tap's offset
//    and padding status are fixed per lane (computed once, 0x80000000 for a padding tap:
//    the buffer range check answers 0) and the channel moves a scalar offset.
// No LDS, no barrier and no address arithmetic in the K loop: a step is one MFMA, one
// dword load and a quarter of a 16-byte load. The loads of chunk i+1 are issued into the
// registers MFMA j of chunk i has just read. The K loop of a tile is shared by the KW
// waves of a workgroup (up to 16, i.e. 1024 threads), whose partial tiles meet in LDS and
// are added in wave order (results do not depend on timing); bias, residual and activation
// ride in that epilogue, so a layer is one launch. Only when a tile's K loop is worth more
// than one workgroup (512->512 on 7x7: 32 tiles) is it also split over workgroups, which
// add into an initialised output with float atomics like the split launches of conv.hip.
#include "conv_params.h"

using namespace pet;
using namespace pet::mfma;

namespace {

template <int TM_, int TN_, int KW_, int RS_>
struct DirectCfg {
    static constexpr int TM = TM_, TN = TN_, KW = KW_, RS = RS_;
    static constexpr int CB = RS == 9 ? 8 : 32; // channels per K chunk
    static constexpr int KC = CB * RS;          // K per chunk
    static constexpr int KH = KC / 2;           // MFMA steps per chunk (k per half-wave)
    static constexpr int CH = CB / 2;           // channels per half-wave
    static constexpr int NQ = KH / 4;           // 16-byte words of A per row and chunk
    static constexpr int NT = 64 * KW;
    static constexpr int PPR = KC / 4;          // 16-byte words per row of a chunk's A tile
    static constexpr int A_LD = KC + 4;         // LDS row stride of the parked tile (floats)
    static constexpr int NREG = TM * TN * 16;
    // LDS per wave: the parked A tile during the K loop, its partial tile afterwards
    static constexpr int WAVE_LDS =
        TM * 32 * A_LD > NREG * 64 ? TM * 32 * A_LD : NREG * 64;
    static constexpr int RPW = NREG / KW;       // accumulator registers a wave finishes
    static_assert(KH % 4 == 0 && NREG % KW == 0 && RPW >= 1 && (32 * PPR) % 64 == 0 &&
                      32 * PPR / 64 == NQ,
                  "bad direct tile");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void conv_direct_kernel(ConvParams p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TM = Cfg::TM, TN = Cfg::TN, KW = Cfg::KW, RS = Cfg::RS;
    constexpr int CB = Cfg::CB, KC = Cfg::KC, KH = Cfg::KH, CH = Cfg::CH;
    constexpr int RPW = Cfg::RPW, NQ = Cfg::NQ, PPR = Cfg::PPR;
    constexpr int A_LD = Cfg::A_LD, WAVE_LDS = Cfg::WAVE_LDS;
    constexpr int SW = RS == 9 ? 3 : 1, SR = RS / SW;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hk = lane >> 5;
    const int g = fd_div(blockIdx.z, p.fd_splitk);
    const int ks = blockIdx.z - g * p.splitk;
    const int m0 = blockIdx.y * (32 * TM);
    const int n0 = blockIdx.x * (32 * TN);
    const int HW = p.H * p.W;
    // strides of a channel, a row and a column of x (a view brings its own)
    const int xsc = p.xv.on ? (int)p.xv.sc : HW;
    const int xsh = p.xv.on ? (int)p.xv.sh : p.W;
    const int xsw = p.xv.on ? (int)p.xv.sw : 1;

    // this wave's share of the K chunks: share ks * KW + wave of splitk * KW
    const int nchunks = p.cpg / CB;
    const int shares = p.splitk * KW;
    const int sh_id = ks * KW + wave;
    const int cb = (int)(((long long)sh_id * nchunks) / shares);
    const int ce = (int)(((long long)(sh_id + 1) * nchunks) / shares);

    // ---- per-lane invariants of the B gather (pad offset folded into the base)
    unsigned voffB[TN][RS];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        const int pix = min(n0 + tn * 32 + l32, p.NPIX - 1);
        const unsigned n = fd_div(pix, p.fd_opix);
        const unsigned rem = pix - n * p.OPIX;
        const unsigned oh = fd_div(rem, p.fd_ow);
        const unsigned ow = rem - oh * p.OW;
        const int ih0 = (int)oh * p.sh, iw0 = (int)ow * p.sw;
        const unsigned pb = (p.xv.on ? view_batch_offset(p.xv, n) : n * (unsigned)(p.C * HW)) +
                            ih0 * xsh + iw0 * xsw + hk * (CH * xsc);
#pragma unroll
        for (int r = 0; r < SR; ++r)
#pragma unroll
            for (int s = 0; s < SW; ++s) {
                const bool ok = (unsigned)(ih0 + r * p.dh - p.ph) < (unsigned)p.H &&
                                (unsigned)(iw0 + s * p.dw - p.pw) < (unsigned)p.W;
                voffB[tn][r * SW + s] = ok ? (pb + r * p.dh * xsh + s * p.dw * xsw) * 4u : kOob;
            }
    }
    const int padoff = p.ph * xsh + p.pw * xsw;
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.x + (long long)g * p.cpg * xsc - padoff);
    // ---- and of the A tile: word i = q * 64 + lane is row i / PPR, floats 4 * (i % PPR) ..
    unsigned voffA[TM][NQ];
    int parkA[NQ]; // where that word is parked in the wave's LDS region (floats)
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int i = q * 64 + lane, row = i / PPR, pc = i - row * PPR;
        parkA[q] = row * A_LD + pc * 4;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            voffA[tm][q] =
                ((unsigned)min(m0 + tm * 32 + row, p.M - 1) * (unsigned)p.K + pc * 4) * 4u;
    }
    float *ldsA = lds + wave * WAVE_LDS;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.w + (p.w_shared ? 0ll : (long long)g * p.M * p.K));

    float a[TM][KH], b[TN][KH];
    uintx4 stage[TM][NQ];
    floatx16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[tm][tn][r] = 0.f;
    const float lo = p.x_relu ? 0.f : -INFINITY; // max(x, lo): ReLU left to this reader, or x

    auto load_a = [&](int q, int chunk) __attribute__((always_inline)) {
        const unsigned so = (unsigned)(chunk * KC) * 4u;
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
            stage[tm][q] = __builtin_amdgcn_raw_buffer_load_b128(ra, voffA[tm][q], so, 0);
    };
    // the staged tile through the wave's LDS region into operand order
    auto park_a = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                *reinterpret_cast<uintx4 *>(ldsA + tm * 32 * A_LD + parkA[q]) = stage[tm][q];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const float4 v = *reinterpret_cast<const float4 *>(
                    ldsA + (tm * 32 + l32) * A_LD + hk * KH + 4 * q);
                a[tm][4 * q] = v.x;
                a[tm][4 * q + 1] = v.y;
                a[tm][4 * q + 2] = v.z;
                a[tm][4 * q + 3] = v.w;
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };
    auto load_b = [&](int j, int chunk) __attribute__((always_inline)) {
        const int cj = j / RS, t = j % RS; // channel inside the half-chunk, tap
        const unsigned so = (unsigned)((chunk * CB + cj) * xsc) * 4u;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            b[tn][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rb, voffB[tn][t], so, 0));
    };
    auto mfma_step = [&](int j) __attribute__((always_inline)) {
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const float bv = fmaxf(b[tn][j], lo);
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][j], bv, acc[tm][tn], 0, 0, 0);
        }
    };

    if (cb < ce) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
            load_a(q, cb);
#pragma unroll
        for (int j = 0; j < KH; ++j)
            load_b(j, cb);
        park_a();
        for (int chunk = cb; chunk + 1 < ce; ++chunk) {
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                load_a(q, chunk + 1);
#pragma unroll
            for (int j = 0; j < KH; ++j) {
                mfma_step(j);
                load_b(j, chunk + 1); // refill what this step has just read
            }
            park_a();
        }
#pragma unroll
        for (int j = 0; j < KH; ++j)
            mfma_step(j);
    }

    // ---- the KW partial tiles meet in LDS: each wave's tile in its own region,
    // [register][lane]
    if (KW > 1) {
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    lds[wave * WAVE_LDS + ((tm * TN + tn) * 16 + r) * 64 + lane] = acc[tm][tn][r];
        __syncthreads();
    }
    const float *__restrict__ bias = (p.bias && p.bias_mode == 1) ? p.bias + g * p.M : nullptr;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int reg = wave * RPW + i; // wave-uniform
        float v = 0.f;
        if (KW > 1) {
#pragma unroll
            for (int w2 = 0; w2 < KW; ++w2)
                v += lds[w2 * WAVE_LDS + reg * 64 + lane];
        } else {
            // KW == 1: the wave keeps its own registers (reg is a compile-time constant)
            v = acc[i / (TN * 16)][(i / 16) % TN][i % 16];
        }
        const int tm = reg / (TN * 16), tn = (reg / 16) % TN, rr = reg % 16;
        const int f = m0 + tm * 32 + (rr / 4) * 8 + hk * 4 + (rr % 4);
        const int pix = n0 + tn * 32 + l32;
        if (f >= p.M || pix >= p.NPIX)
            continue;
        const unsigned n = fd_div(pix, p.fd_opix);
        const unsigned rem = pix - n * p.OPIX;
        long long yi = ((long long)n * p.F + (long long)g * p.M + f) * p.OPIX + rem;
        if (p.yv.on) {
            const unsigned oh = fd_div(rem, p.fd_ow);
            yi = (long long)view_batch_offset(p.yv, n) + ((long long)g * p.M + f) * p.yv.sc +
                 oh * p.yv.sh + (rem - oh * p.OW) * p.yv.sw;
        }
        if (p.atomic_out) {
            // y was initialised (bias, residual) before this launch; activation after it
            if (p.res_first && ks == 0) {
                const float rv = p.res[yi];
                v += p.res_relu ? fmaxf(rv, 0.f) : rv;
            }
            unsafeAtomicAdd(p.y + yi, v);
            continue;
        }
        if (bias)
            v += bias[f];
        if (p.bias && p.bias_mode == 2)
            v += p.bias[(size_t)g * p.bias_gstride + rem];
        if (p.res) {
            const float rv = p.res[yi];
            v += p.res_relu ? fmaxf(rv, 0.f) : rv;
        }
        p.y[yi] = apply_act(v, p.act);
    }
}

// ---- host side ------------------------------------------------------------------------

struct DirectChoice {
    int tm, tn, kw, splitk;
    double cost;
};

// Waves of this tile shape a SIMD holds at once (vector registers: operands of one chunk,
// accumulators, offsets).
int waves_per_simd(int tm, int tn) { return tm * tn == 1 ? 4 : (tm * tn == 2 ? 3 : 2); }

// Cost of a configuration in MFMA cycles on the busiest SIMD, plus what every launch
// pays: the busiest CU runs ceil(workgroups / 256) workgroups, each of which puts KW / 4
// waves on every SIMD, and a wave issues (chunks it owns) * KH * TM * TN MFMAs of 64 cycles;
// loads go through the L1 at about 64 bytes per cycle and CU.
DirectChoice choose_direct(const ConvParams &p, int rs, bool allow_split) {
    const int cbk = rs == 9 ? 8 : 32, kh = cbk * rs / 2;
    const int nchunks = p.cpg / cbk;
    DirectChoice best{0, 0, 0, 1, 1e30};
    static const int kws[3] = {4, 8, 16};
    for (int tm = 1; tm <= 2; ++tm)
        for (int tn = 1; tn <= 2; ++tn)
            for (int kwi = 0; kwi < 3; ++kwi)
                for (int sk = 1; sk <= (allow_split ? 16 : 1); sk *= 2) {
                    const int kw = kws[kwi];
                    if (kw * sk > nchunks && !(kw == 4 && sk == 1))
                        continue; // every wave gets a chunk (the smallest shape is always allowed)
                    const int occ = waves_per_simd(tm, tn);
                    if (kw / 4 > occ)
                        continue;
                    const long long tiles = (long long)((p.M + 32 * tm - 1) / (32 * tm)) *
                                            ((p.NPIX + 32 * tn - 1) / (32 * tn)) * p.G * sk;
                    const int wg_per_cu = std::max(1, (occ * 4) / kw);
                    const long long on_cu = (tiles + 255) / 256; // workgroups of the busiest CU
                    const int chunks = (nchunks + kw * sk - 1) / (kw * sk);
                    const double per_wave = (double)chunks * kh * tm * tn * 64.0;
                    // resident workgroups share the SIMDs; rounds beyond residency queue up
                    const double mfma = (double)on_cu * (kw / 4) * per_wave;
                    const double l1 = (double)on_cu * kw * chunks * kh * (tm + tn) * 256.0 / 64.0;
                    const double rounds = std::ceil((double)on_cu / wg_per_cu);
                    double cost = std::max(mfma, l1) + rounds * 2500.0 + chunks * 300.0;
                    if (sk > 1)
                        cost += 6000.0 + 100.0 * sk; // the initialising and activating launches
                    if (cost < best.cost)
                        best = DirectChoice{tm, tn, kw, sk, cost};
                }
    return best;
}

template <int TM, int TN, int KW, int RS>
int launch_direct_cfg(const ConvParams &p, dim3 grid, hipStream_t stream) {
    using Cfg = DirectCfg<TM, TN, KW, RS>;
    const size_t lds_bytes = (size_t)KW * Cfg::WAVE_LDS * sizeof(float);
    static int attr_status = [&] {
        if (lds_bytes <= 64 * 1024)
            return 0;
        return hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_direct_kernel<Cfg>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds_bytes) == hipSuccess
                   ? 0
                   : 1;
    }();
    if (attr_status)
        return -1;
    hipLaunchKernelGGL((conv_direct_kernel<Cfg>), grid, dim3(Cfg::NT), lds_bytes, stream, p);
    return check_launch("conv_direct_kernel");
}

template <int RS>
int launch_direct_rs(const ConvParams &p, const DirectChoice &c, dim3 grid, hipStream_t stream) {
#define PET_DIRECT_CASE(TM, TN, KW)                                                             \
    if (c.tm == TM && c.tn == TN && c.kw == KW)                                                 \
        return launch_direct_cfg<TM, TN, KW, RS>(p, grid, stream);
    PET_DIRECT_CASE(1, 1, 4)
    PET_DIRECT_CASE(1, 1, 8)
    PET_DIRECT_CASE(1, 1, 16)
    PET_DIRECT_CASE(1, 2, 4)
    PET_DIRECT_CASE(1, 2, 8)
    PET_DIRECT_CASE(2, 1, 4)
    PET_DIRECT_CASE(2, 1, 8)
    PET_DIRECT_CASE(2, 2, 4)
    PET_DIRECT_CASE(2, 2, 8)
#undef PET_DIRECT_CASE
    return -1;
}

} // namespace

namespace pet {
namespace mfma {

int try_launch_direct(const ConvParams &p0, hipStream_t stream) {
    // PET_HIP_DIRECT: 0 never, 1 (default) when the cost model prefers it, 2 whenever it
    // applies. PET_HIP_DIRECT_CFG="tm,tn,kw,splitk" forces a configuration.
    static const int mode = getenv("PET_HIP_DIRECT") ? atoi(getenv("PET_HIP_DIRECT")) : 1;
    if (mode == 0 || p0.static_ws || p0.wpacked)
        return -1;
    if (p0.T != 1 || p0.KT != 1 || p0.pt != 0 || p0.st != 1 || p0.OT != 1)
        return -1;
    const int rs = p0.R * p0.S;
    const bool rs9 = rs == 9 && p0.R == 3 && p0.cpg % 8 == 0;
    const bool rs1 = rs == 1 && p0.cpg % 32 == 0;
    if (!rs9 && !rs1)
        return -1;
    const long long in_bytes = 4ll * p0.N * p0.C * p0.H * p0.W + 4ll * (p0.ph * p0.W + p0.pw);
    const long long w_bytes = 4ll * p0.F * p0.K;
    if (in_bytes >= (1ll << 31) || w_bytes >= (1ll << 31) || ((uintptr_t)p0.w & 15) != 0 ||
        p0.K % 4 != 0)
        return -1;
    // small problems only: beyond a few microseconds of MFMA work the LDS-staged tiles,
    // which read every operand once per 64 rows or columns, win
    const double flop = 2.0 * p0.NPIX * (double)p0.F * p0.K;
    static const double max_gflop =
        getenv("PET_HIP_DIRECT_MAX_GFLOP") ? atof(getenv("PET_HIP_DIRECT_MAX_GFLOP")) : 0.8;
    if (mode == 1 && flop > max_gflop * 1e9)
        return -1;
    ConvParams p = p0;
    const bool allow_split = !deterministic();
    DirectChoice c = choose_direct(p, rs9 ? 9 : 1, allow_split);
    const char *forced = getenv("PET_HIP_DIRECT_CFG"); // read per call: a tuning aid
    if (forced) {
        int tm, tn, kw, sk;
        if (sscanf(forced, "%d,%d,%d,%d", &tm, &tn, &kw, &sk) == 4) {
            c = DirectChoice{tm, tn, kw, std::max(1, sk), 0.0};
            if (!allow_split)
                c.splitk = 1;
        }
    }
    if (p.force_splitk > 0 && allow_split) // the host layer's algorithm search
        c.splitk = p.force_splitk;
    const int nchunks = p.cpg / (rs9 ? 8 : 32);
    c.splitk = std::max(1, std::min(c.splitk, nchunks));
    if (p.w_shared || p.bias_gstride) // the initialising launch knows one bias vector only
        c.splitk = 1;
    const bool exists = (c.tm == 1 || c.tm == 2) && (c.tn == 1 || c.tn == 2) &&
                        (c.kw == 4 || c.kw == 8 || (c.kw == 16 && c.tm * c.tn == 1));
    if (!exists || (long long)p.G * c.splitk > 65535 ||
        (p.M + 32 * c.tm - 1) / (32 * c.tm) > 65535)
        return -1;
    p.splitk = c.splitk;
    p.fd_splitk = make_fastdiv((unsigned)p.splitk);
    p.atomic_out = p.splitk > 1;
    p.streamk = 0;
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
    dim3 grid((p.NPIX + 32 * c.tn - 1) / (32 * c.tn), (p.M + 32 * c.tm - 1) / (32 * c.tm),
              p.G * p.splitk);
    int rc = rs9 ? launch_direct_rs<9>(p, c, grid, stream) : launch_direct_rs<1>(p, c, grid, stream);
    if (rc == PET_HIP_OK && p.atomic_out && p.act != PET_HIP_ACT_NONE &&
        !(p.defer_relu && p.act == PET_HIP_ACT_RELU))
        rc = pet_hip_activation(p.y, p.y, (size_t)p.NPIX * p.F, p.act, (pet_hip_stream_t)stream);
    return rc;
}

} // namespace mfma
} // namespace pet
