// Network stems: 7x7 filters, stride 2, three input channels (ResNet's 7x7/2 on RGB, the
// 3x7x7/(1,2,2) of ResNet3D; ConvOp::compute, src/Graph/operator.cc:94-158, at those
// arguments). With K = 147 per time slice an im2col tile is a gather of single floats with a
// bounds test each, and the general kernel spends more on that gather than on its MFMAs.
// Here a workgroup first copies the input patch its 8 x 16 output pixels read
// (3 x 21 x 37 floats per time slice) and the filter bank (64 x 147) into LDS with coalesced
// loads, one bounds test per patch element; after that every MFMA operand is one LDS read at
// a compile-time offset from a per-lane base, because the K loop is fully unrolled over
// (channel, row, tap):
//   * lane (l32, hk) of a wave holds pixel l32 of the wave's 2 x 16 pixels and k = 2j + hk
//     in step j. The patch offset of tap k is a constant; a lane with hk = 1 needs tap
//     k + 1, which is one float further, or a fixed distance further where k + 1 starts a
//     new filter row or channel: three per-lane base registers, chosen at compile time;
//   * patch rows are 48 floats apart, so the wave's two pixel rows (2 * 48 floats apart)
//     fall into opposite halves of the 64 LDS banks, and filter rows are 150 floats apart
//     (75 odd), so the 32 filters x 2 k of a read spread over all banks.
// K = 147 is odd: the last step's second k reads a zero filter column against a zero cell.
// 3-D: one time slice after the other through the same LDS (a slice outside the clip is
// skipped, every pixel of a workgroup has the same output time); the next slice's loads are
// in flight during this slice's MFMAs. Operands are read from LDS four steps ahead of their
// MFMAs. Measured on MI355X: 1x3x224x224 -> 64 in 8.2 us (general kernel: 14.1),
// 1x3x16x112x112 -> 64, 3x7x7, in 40 us (66). Shader-clock stamps inside the 3-D launch: two
// co-resident workgroups keep the matrix pipes busy through their MFMA phases (57 K cycles
// for the pair); address set-up and the first loads (9 K), three LDS fills (5 K) and the
// stores (5 K) run in lockstep in both and are not hidden. What moved the time: all of a
// slice's loads issued before the first wait (a loop of load -> LDS write was one trip to
// memory per element), 32-bit buffer addressing (registers for two workgroups per CU), the
// bias read from LDS in the epilogue instead of one global load per output. What did not:
// hoisting the index arithmetic out of the slice loop, the read-ahead, 32 filters to a
// workgroup (50 us).
#include "conv_params.h"

namespace pet {
namespace mfma {

namespace {

constexpr int kR = 7, kS = 7, kC = 3, kStride = 2;
constexpr int kTH = 8, kTW = 16;                    // output pixels of a workgroup
constexpr int kPH = (kTH - 1) * kStride + kR;       // 21 patch rows
constexpr int kPWused = (kTW - 1) * kStride + kS;   // 37 patch columns
constexpr int kPW = 48;                             // patch row stride (floats)
constexpr int kPatchPlane = kPH * kPW;
constexpr int kPatch = kC * kPatchPlane;
constexpr int kTaps = kR * kS;                      // 49
constexpr int kK = kC * kTaps;                      // 147
constexpr int kSteps = (kK + 1) / 2;                // 74
constexpr int kLDW = 150;                           // filter row stride (floats)
constexpr int kWs = 64 * kLDW;                      // up to 64 filters to a workgroup
constexpr int kZero = kPatch + kWs;                 // a cell that stays zero
constexpr int kBias = kZero + 4;                     // the workgroup's 64 bias values
constexpr int kLds = kBias + 64;
constexpr int kAhead = 4;                            // MFMA steps between an LDS read and its use
constexpr int kPatchLoads = (kC * kPH * kPWused + 255) / 256;  // per thread and slice
static_assert((2 * kPW) % 64 == 32, "the two pixel rows of a wave must use different banks");
static_assert(kLDW >= kK + 1 && kLDW % 2 == 0 && (kLDW / 2) % 2 == 1, "filter row stride");

constexpr int tap_offset(int k) {
    return ((k / kTaps) * kPH + (k % kTaps) / kS) * kPW + k % kS;
}

template <bool IS3D, int TM>
__global__ __launch_bounds__(256) void conv_stem_kernel(ConvParams p, int tiles_x) {
    constexpr int FB = 32 * TM;                               // filters of a workgroup
    __shared__ __attribute__((aligned(16))) float lds[kLds];
    float *patch = lds, *ws = lds + kPatch;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hk = lane >> 5;

    const int ty = blockIdx.x / tiles_x, tx = blockIdx.x - ty * tiles_x;
    const int oh0 = ty * kTH, ow0 = tx * kTW;
    const int f0 = blockIdx.y * FB;
    const int n = IS3D ? blockIdx.z / p.OT : blockIdx.z;
    const int ot = IS3D ? blockIdx.z - n * p.OT : 0;
    const int HW = p.H * p.W;
    const int ih0 = oh0 * kStride - p.ph, iw0 = ow0 * kStride - p.pw;

    // the filter rows' zero column and the zero cell, once (no slice writes them)
    if (tid < FB)
        ws[tid * kLDW + kK] = 0.f;
    if (tid == 0)
        lds[kZero] = 0.f;
    if (tid < FB) // the epilogue reads its bias from LDS: a load per output would be a trip each
        lds[kBias + tid] = p.bias ? p.bias[min(f0 + tid, p.F - 1)] : 0.f;

    floatx16 acc[TM];
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[tm][r] = 0.f;

    // per-lane bases, in floats: pixel (py, px) of the tile, tap k + hk
    const int py = wave * 2 + (l32 >> 4), px = l32 & 15;
    const int pix = py * kStride * kPW + px * kStride;
    const int b_next = pix + hk;                                       // k + 1 in the same row
    const int b_row = pix + hk * (kPW - (kS - 1));                     // k + 1 starts a row
    const int b_chan = pix + hk * (kPatchPlane - (kR - 1) * kPW - (kS - 1)); // ... a channel
    const int b_last = hk ? kZero - tap_offset(kK - 1) : pix;          // k + 1 does not exist
    const int a_base = kPatch + l32 * kLDW + hk;

    // A slice's patch [c][y][x] (zero outside the image) and filters (rows of 147,
    // [f][c][r][s]) travel through registers: every load of a slice is issued before anything
    // waits for one, and the next slice's loads fly during this slice's MFMAs. 32-bit buffer
    // addressing: an offset of 2^31 reads as zero, which is the padding. Nothing in a load's
    // address but a scalar base depends on the slice, so the offsets are worked out once:
    // patch element e = tid + 256 i; filter element (f, k) = (16 wave' + i, lane + 64 kk),
    // a wave reading 64 consecutive k of one filter row.
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.x), rw = make_rsrc(p.w);
    unsigned p_off[kPatchLoads];
    int p_lds[kPatchLoads];
#pragma unroll
    for (int i = 0; i < kPatchLoads; ++i) {
        const int e = tid + i * 256;
        const int c = e / (kPH * kPWused);
        const int rem = e - c * (kPH * kPWused);
        const int y = rem / kPWused, x = rem - y * kPWused;
        const int ih = ih0 + y, iw = iw0 + x;
        const bool ok = e < kC * kPH * kPWused && (unsigned)ih < (unsigned)p.H &&
                        (unsigned)iw < (unsigned)p.W;
        p_off[i] = ok ? (unsigned)(c * p.T * HW + ih * p.W + iw) * 4u : kOob;
        p_lds[i] = e < kC * kPH * kPWused ? (c * kPH + y) * kPW + x : -1;
    }
    constexpr int kKChunks = (kK + 63) / 64;                  // 3
    constexpr int kRowsPerWave = FB / 4;
    unsigned w_off[kKChunks];
#pragma unroll
    for (int kk = 0; kk < kKChunks; ++kk) {
        const int k = lane + 64 * kk;
        const int c = k / kTaps, t = k - c * kTaps;
        w_off[kk] = k < kK ? (unsigned)(c * p.KT * kTaps + t) * 4u : kOob;
    }
    const int w_lds = kPatch + wave * kRowsPerWave * kLDW + lane;
    float pv[kPatchLoads], wv[kRowsPerWave][kKChunks];
    auto time_of = [&](int q) { return IS3D ? ot * p.st - p.pt + q * p.dt : 0; };
    auto next_slice = [&](int q) { // the first slice from q on that lies inside the clip
        while (q < p.KT && (unsigned)time_of(q) >= (unsigned)p.T)
            ++q;
        return q;
    };
    auto load_slice = [&](int q) __attribute__((always_inline)) {
        const unsigned x_slice = (unsigned)(((size_t)n * p.C * p.T + time_of(q)) * HW) * 4u;
#pragma unroll
        for (int i = 0; i < kPatchLoads; ++i)
            pv[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rx, p_off[i], x_slice, 0));
#pragma unroll
        for (int i = 0; i < kRowsPerWave; ++i) {
            const int fg = min(f0 + wave * kRowsPerWave + i, p.F - 1);
            const unsigned row = (unsigned)(fg * p.K + q * kTaps) * 4u; // wave-uniform
#pragma unroll
            for (int kk = 0; kk < kKChunks; ++kk)
                wv[i][kk] =
                    __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rw, w_off[kk], row, 0));
        }
    };
    auto park_slice = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kPatchLoads; ++i)
            if (p_lds[i] >= 0)
                patch[p_lds[i]] = p.x_relu ? fmaxf(pv[i], 0.f) : pv[i];
#pragma unroll
        for (int i = 0; i < kRowsPerWave; ++i)
#pragma unroll
            for (int kk = 0; kk < kKChunks; ++kk)
                if (lane + 64 * kk < kK)
                    lds[w_lds + i * kLDW + 64 * kk] = wv[i][kk];
    };

    int q = next_slice(0);
    if (q < p.KT)
        load_slice(q);
    while (q < p.KT) {
        park_slice();
        __syncthreads();
        q = next_slice(q + 1);
        if (q < p.KT)
            load_slice(q);
        // operands are read kAhead steps before their MFMAs, through a ring of register sets;
        // the scheduling barriers keep the compiler from sinking a read down to its use
        float av[kAhead][TM], bv[kAhead];
        auto read_step = [&](int j, int set) __attribute__((always_inline)) {
            const int k0 = 2 * j;
            const int s0 = k0 % kS, r0 = (k0 % kTaps) / kS;
            const int off = tap_offset(k0);
            if (k0 + 1 >= kK)
                bv[set] = lds[b_last + off];
            else if (s0 < kS - 1)
                bv[set] = patch[b_next + off];
            else if (r0 < kR - 1)
                bv[set] = patch[b_row + off];
            else
                bv[set] = patch[b_chan + off];
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                av[set][tm] = lds[a_base + tm * 32 * kLDW + k0];
        };
#pragma unroll
        for (int j = 0; j < kAhead; ++j)
            read_step(j, j);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
#pragma unroll
            for (int tm = 0; tm < TM; ++tm)
                acc[tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j % kAhead][tm], bv[j % kAhead],
                                                               acc[tm], 0, 0, 0);
            if (j + kAhead < kSteps)
                read_step(j + kAhead, j % kAhead);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (q < p.KT)
            __syncthreads(); // this slice's reads are over before the next one is parked
    }

    // ---- epilogue: register r of tile tm is filter tm*32 + (r/4)*8 + hk*4 + r%4, pixel l32
    const int oh = oh0 + py, ow = ow0 + px;
    if (oh >= p.OH || ow >= p.OW)
        return;
    const size_t plane = (size_t)p.OH * p.OW;
    const unsigned fstride = (unsigned)(p.OT * plane); // floats between filters of the output
    float *yb = p.y + ((size_t)n * p.F * p.OT + ot) * plane + (size_t)oh * p.OW + ow +
                (size_t)(f0 + hk * 4) * fstride;
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int fl = tm * 32 + (r / 4) * 8 + (r % 4); // + hk * 4: this lane's filter
            if (f0 + fl + hk * 4 < p.F)
                yb[(unsigned)fl * fstride] =
                    apply_act(acc[tm][r] + lds[kBias + fl + hk * 4], p.act);
        }
}

} // namespace

// Returns -1 when the kernel does not apply (the caller goes on to the general kernel).
int try_launch_stem(const ConvParams &p, hipStream_t stream) {
    static const bool off = getenv("PET_HIP_STEM") && atoi(getenv("PET_HIP_STEM")) == 0;
    if (off || p.G != 1 || p.C != kC || p.R != kR || p.S != kS || p.sh != kStride ||
        p.sw != kStride || p.dh != 1 || p.dw != 1 || p.res || p.bias_mode == 2 || p.w_shared ||
        p.wpacked || p.y_init)
        return -1;
    if (4ll * p.N * p.C * p.T * p.H * p.W >= (1ll << 31) || 4ll * p.F * p.K >= (1ll << 31))
        return -1; // the loads address with 32-bit byte offsets
    const bool is3d = p.T > 1 || p.KT > 1 || p.pt > 0 || p.st > 1;
    const long long planes = (long long)p.N * p.OT;
    const int tiles_x = (p.OW + kTW - 1) / kTW, tiles_y = (p.OH + kTH - 1) / kTH;
    if (planes > 65535 || (long long)tiles_x * tiles_y >= (1ll << 31))
        return -1;
    // 64 filters to a workgroup, or 32 while that leaves CUs without one
    const long long wgs64 = (long long)tiles_x * tiles_y * planes * ((p.F + 63) / 64);
    const int tm = (p.F > 32 && wgs64 >= 256) ? 2 : 1;
    const dim3 grid((unsigned)(tiles_x * tiles_y), (unsigned)((p.F + 32 * tm - 1) / (32 * tm)),
                    (unsigned)planes);
    if (grid.y > 65535)
        return -1;
    if (is3d) {
        if (tm == 2)
            hipLaunchKernelGGL((conv_stem_kernel<true, 2>), grid, dim3(256), 0, stream, p, tiles_x);
        else
            hipLaunchKernelGGL((conv_stem_kernel<true, 1>), grid, dim3(256), 0, stream, p, tiles_x);
    } else {
        if (tm == 2)
            hipLaunchKernelGGL((conv_stem_kernel<false, 2>), grid, dim3(256), 0, stream, p, tiles_x);
        else
            hipLaunchKernelGGL((conv_stem_kernel<false, 1>), grid, dim3(256), 0, stream, p, tiles_x);
    }
    return check_launch("conv_stem_kernel");
}

} // namespace mfma
} // namespace pet
