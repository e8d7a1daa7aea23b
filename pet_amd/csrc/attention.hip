// Multi-head attention core in one launch: for every head,
//     out = softmax(scale * Q K^T) V
// with Q, K, V read straight from the [seq, heads*dh] activations of the projection
// matmuls (head h is columns h*dh .. h*dh+dh-1) and out written in the same layout. In
// the operator graph this is Transpose (head split) x 3 -> Matmul(transB) -> Mul(scale) ->
// Softmax -> Matmul -> Transpose (head merge) -> Reshape: eight launches, four of them
// pure layout moves. The reference runs the two products through cuBLAS and the softmax
// through an inline kernel (src/Graph/code_engine.cc:1103-1169, 1707-1731).
//
// One workgroup owns 32 queries of one head; wave w owns keys 32w .. 32w+31:
//   S_w^T = K_w Q_blk^T   32x32 tile, both operands contiguous along dh (16-byte loads). The
//                         transposed product leaves a lane holding ONE query (its column)
//                         and 16 of the 32 keys in its accumulator registers, so
//   row max and row sum   are 16 in-register steps and one exchange between the half-waves,
//                         then across waves through LDS, and
//   O_w = P_w V_w         takes the accumulator registers directly as its row operand:
//                         register r of half-wave hk is key (r/4)*8 + hk*4 + r%4, and the MFMA
//                         steps are free to take the keys in that order; V is read across
//                         lanes along dh (coalesced), and its loads are issued before the
//                         first product so that they are there when the softmax is done.
//   out = (sum_w O_w) / rowsum: the waves add their tiles into four LDS slots, wave w into
//   slot w % 4 in rounds of four waves, and the slots are added in order (results do not
//   depend on timing).
// seq <= 512 (16 waves), dh a multiple of 32 up to 128.
#include "mfma_common.h"

using namespace pet;
using namespace pet::mfma;

namespace {

struct AttnParams {
    const float *q, *k, *v;
    float *out;
    const float *scale_dev;
    float scale;
    int batch, heads, seq;
    int ldq, ldk, ldv, ldo;          // row strides in floats
    long long sq, sk, sv, so;        // batch strides in floats
};

constexpr int kSlots = 4; // partial output tiles in LDS

// MAXT: 256 for up to four waves (seq <= 128; registers are plentiful), else 1024, where a
// wave has 128 registers: V is then fetched after the softmax for dh > 64, and a 128-wide
// head takes its S product in two halves.
template <int DH, int MAXT>
__global__ __launch_bounds__(MAXT) void attention_kernel(AttnParams p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int TN = DH / 32;
    constexpr int KH = DH / 2; // dh values per half-wave in the S product
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nw = blockDim.x >> 6;
    const int l32 = lane & 31, hk = lane >> 5;
    const int q0 = blockIdx.x * 32;
    const int head = blockIdx.y;
    const int b = blockIdx.z;
    const int k0 = wave * 32;
    // LDS: [red: nw*32][sumred: nw*32][O slots: kSlots*32*DH]
    float *red = lds;
    float *sred = lds + nw * 32;
    float *obuf = lds + 2 * nw * 32;

    const float scale = p.scale * (p.scale_dev ? *p.scale_dev : 1.f);
    const float *qp = p.q + b * p.sq + (size_t)min(q0 + l32, p.seq - 1) * p.ldq + head * DH + hk * KH;
    const float *kp = p.k + b * p.sk + (size_t)min(k0 + l32, p.seq - 1) * p.ldk + head * DH + hk * KH;
    constexpr bool EARLY_V = MAXT == 256 || DH <= 64;
    constexpr int NJ = KH / 4, CJ = (MAXT == 1024 && NJ > 8) ? 8 : NJ; // float4 per operand and pass
    float4 qv[CJ], kv[CJ];
#pragma unroll
    for (int j = 0; j < CJ; ++j) {
        qv[j] = *reinterpret_cast<const float4 *>(qp + 4 * j);
        kv[j] = *reinterpret_cast<const float4 *>(kp + 4 * j);
    }
    // V rows of this wave's keys in the order the accumulator registers hold them
    const float *vp = p.v + b * p.sv + head * DH + l32;
    float vv[16][TN];
    auto load_v = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = k0 + (r / 4) * 8 + hk * 4 + (r % 4);
            const float *vrow = vp + (size_t)min(key, p.seq - 1) * p.ldv;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                vv[r][tn] = vrow[tn * 32];
        }
    };
    if (EARLY_V)
        load_v();

    // S^T: rows = keys (operand A = K), columns = queries (operand B = Q)
    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        s[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NJ; c += CJ) {
        if (c > 0) {
#pragma unroll
            for (int j = 0; j < CJ; ++j) {
                qv[j] = *reinterpret_cast<const float4 *>(qp + 4 * (c + j));
                kv[j] = *reinterpret_cast<const float4 *>(kp + 4 * (c + j));
            }
        }
#pragma unroll
        for (int j = 0; j < CJ; ++j) {
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[j].x, qv[j].x, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[j].y, qv[j].y, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[j].z, qv[j].z, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[j].w, qv[j].w, s, 0, 0, 0);
        }
    }
    // register r of a lane: key k0 + (r/4)*8 + hk*4 + r%4, query q0 + l32
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const bool kvalid = k0 + (r / 4) * 8 + hk * 4 + (r % 4) < p.seq;
        s[r] = kvalid ? s[r] * scale : -INFINITY;
        mx = fmaxf(mx, s[r]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    if (hk == 0)
        red[wave * 32 + l32] = mx;
    __syncthreads();
    float m = red[l32];
    for (int w = 1; w < nw; ++w)
        m = fmaxf(m, red[w * 32 + l32]);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        // a key past the end holds -inf: exp gives 0 (m is finite: key 0 is always valid)
        s[r] = expf(s[r] - m);
        sum += s[r];
    }
    sum += __shfl_xor(sum, 32);
    if (hk == 0)
        sred[wave * 32 + l32] = sum;
    if (!EARLY_V)
        load_v();

    // O_w = P_w V_w: MFMA step r takes key (r/4)*8 + hk*4 + r%4 from both operands
    floatx16 o[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            o[tn][r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r)
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            o[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(s[r], vv[r][tn], o[tn], 0, 0, 0);

    // the waves' O tiles into the slots, a round of kSlots waves at a time
    float *slot = obuf + (wave % kSlots) * (32 * DH);
    for (int round = 0; round * kSlots < nw; ++round) {
        if (wave / kSlots == round) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = (r / 4) * 8 + hk * 4 + (r % 4);
                    float *dst = slot + row * DH + tn * 32 + l32;
                    *dst = round == 0 ? o[tn][r] : *dst + o[tn][r];
                }
        }
        __syncthreads();
    }
    const int nslots = nw < kSlots ? nw : kSlots;
    // out[q0 + row][head*DH + d] = O / rowsum
    for (int i = threadIdx.x; i < 32 * DH; i += blockDim.x) {
        const int row = i / DH, d = i - row * DH;
        if (q0 + row >= p.seq)
            continue;
        float t = sred[row];
        for (int w = 1; w < nw; ++w)
            t += sred[w * 32 + row];
        float v = obuf[i];
        for (int sl = 1; sl < nslots; ++sl)
            v += obuf[sl * (32 * DH) + i];
        p.out[b * p.so + (size_t)(q0 + row) * p.ldo + head * DH + d] = v / t;
    }
}

template <int DH, int MAXT>
int launch_attention_as(const AttnParams &p, hipStream_t stream) {
    const int nw = (p.seq + 31) / 32;
    const size_t lds_bytes = sizeof(float) * (2 * nw * 32 + kSlots * 32 * DH);
    static int attr_status = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(&attention_kernel<DH, MAXT>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   96 * 1024) == hipSuccess
                   ? 0
                   : 1;
    }();
    if (attr_status)
        return set_error(PET_HIP_ERR_RUNTIME, "attention: cannot size the LDS allocation");
    dim3 grid((unsigned)nw, (unsigned)p.heads, (unsigned)p.batch);
    hipLaunchKernelGGL((attention_kernel<DH, MAXT>), grid, dim3(64 * nw), lds_bytes, stream, p);
    return check_launch("attention_kernel");
}

template <int DH>
int launch_attention(const AttnParams &p, hipStream_t stream) {
    return p.seq <= 128 ? launch_attention_as<DH, 256>(p, stream)
                        : launch_attention_as<DH, 1024>(p, stream);
}

} // namespace

extern "C" {

int pet_hip_attention_f32(const float *q, const float *k, const float *v, float *out, int batch,
                          int heads, int seq, int dh, int ldq, int ldk, int ldv, int ldo,
                          long long stride_q, long long stride_k, long long stride_v,
                          long long stride_o, float scale, const float *scale_dev,
                          pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (batch < 0 || heads <= 0 || seq <= 0 || dh <= 0)
        return set_error(PET_HIP_ERR_INVALID, "attention: bad shape");
    if (batch == 0)
        return PET_HIP_OK; // no sequences
    if (!q || !k || !v || !out)
        return set_error(PET_HIP_ERR_INVALID, "attention: null operand");
    const int width = heads * dh;
    if (ldq < width || ldk < width || ldv < width || ldo < width)
        return set_error(PET_HIP_ERR_INVALID, "attention: row stride below heads * dh");
    if (seq > 512 || (dh != 32 && dh != 64 && dh != 96 && dh != 128) || heads > 65535 ||
        batch > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "attention: seq %d (at most 512), head size %d (32, 64, 96 or 128)", seq,
                         dh);
    if ((ldq | ldk) % 4 != 0 || ((uintptr_t)q & 15) || ((uintptr_t)k & 15) || stride_q % 4 != 0 ||
        stride_k % 4 != 0)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "attention: Q and K rows must be 16-byte aligned");
    AttnParams p{q,   k,   v,   out, scale_dev, scale,    batch,    heads,    seq,
                 ldq, ldk, ldv, ldo, stride_q,  stride_k, stride_v, stride_o};
    hipStream_t st = as_stream(stream);
    switch (dh) {
    case 32:
        return launch_attention<32>(p, st);
    case 64:
        return launch_attention<64>(p, st);
    case 96:
        return launch_attention<96>(p, st);
    default:
        return launch_attention<128>(p, st);
    }
}

} // extern "C"
