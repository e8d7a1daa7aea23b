// fp32 MFMA batched matmul for gfx950: C[b] = op(A[b]) * op(B[b]), row-major,
// fused bias (per output column) + activation. Same LDS layouts and MFMA feeding
// as the convolution kernels (A as [m][k], B as [k][n]).
#include "mfma_common.h"

using namespace pet;
using namespace pet::mfma;

namespace {

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
    for (int kt = 0; kt < nk - 1; ++kt) {
        float *cur = lds + (kt & 1) * Cfg::STAGE;
        float *nxt = lds + ((kt + 1) & 1) * Cfg::STAGE;
        load_tiles((kt + 1) * Cfg::BK);
        __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMA block
        mma_block<Cfg>(cur, cur + Cfg::A_ELEMS, acc, wm0, wn0, lane);
        __builtin_amdgcn_sched_barrier(0);
        store_tiles(nxt);
        __syncthreads();
    }
    {
        float *cur = lds + ((nk - 1) & 1) * Cfg::STAGE;
        mma_block<Cfg>(cur, cur + Cfg::A_ELEMS, acc, wm0, wn0, lane);
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

// 0: 128x128, 1: 64x128, 2: 64x64, 3: 32x64
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

} // namespace

namespace {

int bmm_common(int transA, int transB, int b, int m, int n, int k, const float *A, const float *B,
               float *C, const float *bias, const float *res, int act, pet_hip_stream_t stream,
               unsigned flags = 0, int *dry = nullptr) {
    if (flags & ~(unsigned)(PET_HIP_CALL_Y_INITIALISED | PET_HIP_CALL_A_SHARED |
                            PET_HIP_CALL_BIAS_PER_BATCH | 0xff00u))
        return set_error(PET_HIP_ERR_INVALID,
                         "matmul takes PET_HIP_CALL_Y_INITIALISED, PET_HIP_CALL_A_SHARED, "
                         "PET_HIP_CALL_BIAS_PER_BATCH and an algorithm only");
    const unsigned addressing = flags & (PET_HIP_CALL_A_SHARED | PET_HIP_CALL_BIAS_PER_BATCH);
    if (((flags >> 8) & 0xffu) >= PET_HIP_CONV_ALGO_COUNT)
        return set_error(PET_HIP_ERR_INVALID, "unknown algorithm %u", (flags >> 8) & 0xffu);
    if (dry) {
        *dry = 0;
        A = B = reinterpret_cast<const float *>(uintptr_t(256));
        C = reinterpret_cast<float *>(uintptr_t(512));
    }
    if (b < 0 || m < 0 || n < 0 || k < 0)
        return set_error(PET_HIP_ERR_INVALID, "negative matmul dims");
    if (act < PET_HIP_ACT_NONE || act > PET_HIP_ACT_GELU)
        return set_error(PET_HIP_ERR_INVALID, "unknown activation %d", act);
    if ((long long)b * m * n == 0)
        return PET_HIP_OK;
    if (!C)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    if (res == C)
        return set_error(PET_HIP_ERR_INVALID, "the residual must not be the output buffer");
    const size_t cn = (size_t)b * m * n;
    if (k == 0 && dry)
        return PET_HIP_OK;
    if (k == 0) {
        // empty contraction: C = act(bias + residual)
        int rc = res ? pet_hip_memcpy_d2d(C, res, cn * sizeof(float), stream)
                     : pet_hip_fill_f32(C, 0.f, cn, stream);
        if (rc == PET_HIP_OK && (bias || act != PET_HIP_ACT_NONE))
            rc = pet_hip_bias_act(C, bias, C, (size_t)b * m, (size_t)n, 1, act, stream);
        return rc;
    }
    if (!A || !B)
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
    p.act = res ? PET_HIP_ACT_NONE : act;
    if (!transA && !transB) {
        int rc = bmm_as_grouped_1x1(A, B, C, bias, res, b, m, n, k, act, as_stream(stream), flags,
                                    dry);
        if (rc >= 0)
            return rc;
    }
    if (addressing) {
        // no kernel with that addressing applies: one product per batch entry
        for (int i = 0; i < b; ++i) {
            const float *Ai = (flags & PET_HIP_CALL_A_SHARED) ? A : A + (size_t)i * m * k;
            const float *bi = bias && (flags & PET_HIP_CALL_BIAS_PER_BATCH) ? bias + (size_t)i * n
                                                                            : bias;
            int rc = bmm_common(transA, transB, 1, m, n, k, Ai, B + (size_t)i * k * n,
                                C + (size_t)i * m * n, bi, res ? res + (size_t)i * m * n : nullptr,
                                act, stream, flags & ~addressing, dry);
            if (rc != PET_HIP_OK || dry)
                return rc;
        }
        return PET_HIP_OK;
    }
    if (dry) // the general kernel never accumulates into C
        return PET_HIP_OK;
    // the general kernel has no residual operand: add it, and apply the activation,
    // in two small launches afterwards
    auto finish = [&](int rc) {
        if (rc != PET_HIP_OK || !res)
            return rc;
        const float *ins[2] = {C, res};
        const size_t sizes[2] = {cn, cn};
        rc = pet_hip_eltwise(PET_HIP_ADD, ins, sizes, 2, C, cn, stream);
        if (rc == PET_HIP_OK && act != PET_HIP_ACT_NONE)
            rc = pet_hip_activation(C, C, cn, act, stream);
        return rc;
    };
    // float4 loads need every row start 16-byte aligned on both operands
    long long lda = transA ? m : k, ldb = transB ? k : n;
    bool vec = lda % 4 == 0 && ldb % 4 == 0 && p.sA % 4 == 0 && p.sB % 4 == 0 &&
               (((uintptr_t)A | (uintptr_t)B) & 15) == 0 &&
               (transA ? m % 4 == 0 : k % 4 == 0) && (transB ? k % 4 == 0 : n % 4 == 0);
    hipStream_t s = as_stream(stream);
    if (transA)
        return finish(transB ? launch_bmm_t<true, true>(p, b, vec, s)
                             : launch_bmm_t<true, false>(p, b, vec, s));
    return finish(transB ? launch_bmm_t<false, true>(p, b, vec, s)
                         : launch_bmm_t<false, false>(p, b, vec, s));
}

} // namespace

extern "C" {

int pet_hip_bmm_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                    const float *B, float *C, const float *bias, int act,
                    pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return bmm_common(transA, transB, b, m, n, k, A, B, C, bias, nullptr, act, stream);
}

int pet_hip_bmm_res_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                        const float *B, float *C, const float *bias, const float *residual,
                        int act, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return bmm_common(transA, transB, b, m, n, k, A, B, C, bias, residual, act, stream);
}

int pet_hip_bmm_ex_f32(int transA, int transB, int b, int m, int n, int k, const float *A,
                       const float *B, float *C, const float *bias, const float *residual, int act,
                       unsigned flags, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    return bmm_common(transA, transB, b, m, n, k, A, B, C, bias, residual, act, stream, flags);
}

int pet_hip_bmm_accumulates(int transA, int transB, int b, int m, int n, int k, int *yes) {
    PET_REQUIRE_INIT();
    if (!yes)
        return set_error(PET_HIP_ERR_INVALID, "null result pointer");
    return bmm_common(transA, transB, b, m, n, k, nullptr, nullptr, nullptr, nullptr, nullptr,
                      PET_HIP_ACT_NONE, nullptr, 0, yes);
}

} // extern "C"
