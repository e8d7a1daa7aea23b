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
//   S_w = Q_blk K_w^T     32x32 tile, both operands contiguous along dh (16-byte loads)
//   row max and row sum   across the 32 lanes of a half-wave, then across waves through LDS
//   O_w = P_w V_w         P_w goes through LDS to become the row operand; V is read
//                         across lanes along dh (coalesced)
//   out = (sum_w O_w) / rowsum, the waves adding in wave order (results do not depend on
//   timing).
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

template <int DH>
__global__ __launch_bounds__(1024) void attention_kernel(AttnParams p) {
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
    // LDS: [red: nw*32][sumred: nw*32][P: nw*32*33][O: 32*DH]
    float *red = lds;
    float *sred = lds + nw * 32;
    float *pbuf = lds + 2 * nw * 32 + wave * (32 * 33);
    float *obuf = lds + 2 * nw * 32 + nw * (32 * 33);

    const float scale = p.scale * (p.scale_dev ? *p.scale_dev : 1.f);
    const float *qp = p.q + b * p.sq + (size_t)min(q0 + l32, p.seq - 1) * p.ldq + head * DH + hk * KH;
    const float *kp = p.k + b * p.sk + (size_t)min(k0 + l32, p.seq - 1) * p.ldk + head * DH + hk * KH;

    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        s[r] = 0.f;
#pragma unroll
    for (int j = 0; j < KH; j += 4) {
        const float4 a = *reinterpret_cast<const float4 *>(qp + j);
        const float4 bb = *reinterpret_cast<const float4 *>(kp + j);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bb.x, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bb.y, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, bb.z, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, bb.w, s, 0, 0, 0);
    }
    // register r of a lane: query row (r/4)*8 + hk*4 + r%4, key column k0 + l32
    const bool kvalid = k0 + l32 < p.seq;
    float mx[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        s[r] = kvalid ? s[r] * scale : -INFINITY;
        float m = s[r];
#pragma unroll
        for (int off = 1; off < 32; off <<= 1)
            m = fmaxf(m, __shfl_xor(m, off));
        mx[r] = m;
    }
    if (l32 == 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
            red[wave * 32 + (r / 4) * 8 + hk * 4 + (r % 4)] = mx[r];
    }
    __syncthreads();
    float sum[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = (r / 4) * 8 + hk * 4 + (r % 4);
        float m = red[row];
        for (int w = 1; w < nw; ++w)
            m = fmaxf(m, red[w * 32 + row]);
        const float e = kvalid ? expf(s[r] - m) : 0.f;
        s[r] = e;
        float t = e;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1)
            t += __shfl_xor(t, off);
        sum[r] = t;
        pbuf[row * 33 + l32] = e; // P_w as [query][key]
    }
    if (l32 == 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
            sred[wave * 32 + (r / 4) * 8 + hk * 4 + (r % 4)] = sum[r];
    }
    // O_w = P_w V_w: row operand from LDS (this wave's own region), V across lanes
    floatx16 o[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            o[tn][r] = 0.f;
    const float *vp = p.v + b * p.sv + head * DH + l32;
    // the wave's LDS writes above are visible to its own lanes after this wait
    __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const int kk = hk * 16 + j; // key inside the wave's 32
        const float a = pbuf[l32 * 33 + kk];
        const float *vrow = vp + (size_t)min(k0 + kk, p.seq - 1) * p.ldv;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn)
            o[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, vrow[tn * 32], o[tn], 0, 0, 0);
    }
    // sum of the waves' O tiles in wave order
    for (int w = 0; w < nw; ++w) {
        if (wave == w) {
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = (r / 4) * 8 + hk * 4 + (r % 4);
                    float *dst = obuf + row * DH + tn * 32 + l32;
                    *dst = w == 0 ? o[tn][r] : *dst + o[tn][r];
                }
        }
        __syncthreads();
    }
    // out[q0 + row][head*DH + d] = O / rowsum
    for (int i = threadIdx.x; i < 32 * DH; i += blockDim.x) {
        const int row = i / DH, d = i - row * DH;
        if (q0 + row >= p.seq)
            continue;
        float t = sred[row];
        for (int w = 1; w < nw; ++w)
            t += sred[w * 32 + row];
        p.out[b * p.so + (size_t)(q0 + row) * p.ldo + head * DH + d] = obuf[i] / t;
    }
}

template <int DH>
int launch_attention(const AttnParams &p, hipStream_t stream) {
    const int nw = (p.seq + 31) / 32;
    const size_t lds_bytes = sizeof(float) * (2 * nw * 32 + nw * 32 * 33 + 32 * DH);
    static int attr_status = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void *>(&attention_kernel<DH>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                   96 * 1024) == hipSuccess
                   ? 0
                   : 1;
    }();
    if (attr_status)
        return set_error(PET_HIP_ERR_RUNTIME, "attention: cannot size the LDS allocation");
    dim3 grid((unsigned)nw, (unsigned)p.heads, (unsigned)p.batch);
    hipLaunchKernelGGL((attention_kernel<DH>), grid, dim3(64 * nw), lds_bytes, stream, p);
    return check_launch("attention_kernel");
}

} // namespace

extern "C" {

int pet_hip_attention_f32(const float *q, const float *k, const float *v, float *out, int batch,
                          int heads, int seq, int dh, int ldq, int ldk, int ldv, int ldo,
                          long long stride_q, long long stride_k, long long stride_v,
                          long long stride_o, float scale, const float *scale_dev,
                          pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    if (!q || !k || !v || !out)
        return set_error(PET_HIP_ERR_INVALID, "attention: null operand");
    if (batch <= 0 || heads <= 0 || seq <= 0 || dh <= 0)
        return set_error(PET_HIP_ERR_INVALID, "attention: bad shape");
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
