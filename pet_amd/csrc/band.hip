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
//    along k) and stores the part of each tile that lies in the band: a lane's 32 columns r'
//    are 32 consecutive j of one output row, a coalesced store.
//  * GBMML is a GEMM whose K axis runs over r' in [i0' - w, i0' + 31 + w]: the band operand
//    is contiguous along j (zero outside the band), the general operand is read across
//    lanes along n (coalesced).
// Each has a staged kernel (operand tiles read as whole cache lines and turned into operand
// order through a wave-private LDS tile, 32-bit buffer addressing); G2BMM keeps a general
// kernel for feature lengths that are not a multiple of 32 or unaligned operands. Measured
// on 12 x 4096 x 64, w = 256: G2BMM 55 us, GBMML 50 us (3.2 GFLOP each; 100 MB of band
// matrix written resp. read, 13 us at the HBM peak). What moved the time: 64-bit address
// arithmetic and branches out of the epilogue (a tile has only 32 MFMAs at k = 64), and for
// GBMML enough waves (32-column tiles, four waves sharing a tile's K axis). What did not:
// more column tiles per wave, XCD-contiguous order, deeper load batching, prefetching the
// next chunk across the MFMAs.
#include "conv_params.h"
#include <type_traits>

using namespace pet;
using namespace pet::mfma;

namespace {

struct BandParams {
    const float *A, *B;
    float *C;
    int bs, m, k, w, d, n; // k: G2BMM feature length; n: GBMML output columns
    int mc;                // rows per residue class, rounded up: ceil(m / d)
    int rtiles;            // G2BMM: column tiles per row block
    int gx, gy, total, per_xcd; // logical grid, see band_position
    FastDiv fd_gx, fd_gy, fd_d;
};

// Workgroups reach the 8 XCDs round-robin in launch order and every XCD has its own L2. The
// launch is one-dimensional and padded to a multiple of 8; workgroup L takes logical
// position (L % 8) * per + L / 8, so that an XCD walks one contiguous run of (batch, row
// block) pairs and the sliding window of B rows it needs stays in its L2.
// (per_wave: every wave of the workgroup takes a position of its own; else the workgroup
// shares one.)
__device__ __forceinline__ bool band_position(const BandParams &p, int &bx, int &by, int &bz,
                                              bool per_wave = true) {
    const unsigned L = blockIdx.x;
    unsigned logical = (L & 7u) * (unsigned)p.per_xcd + (L >> 3);
    if (per_wave)
        logical = logical * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (logical >= (unsigned)p.total)
        return false;
    const unsigned rest = fd_div(logical, p.fd_gx);
    bx = (int)(logical - rest * (unsigned)p.gx);
    bz = (int)fd_div(rest, p.fd_gy);
    by = (int)(rest - (unsigned)bz * (unsigned)p.gy);
    return true;
}

// General form (any k, any alignment). Logical grid: x = group of TNT r' tiles, y = i' block,
// z = batch * d + rho; a wave keeps its 32 rows of A for TNT column tiles and loads straight
// into operand order (a 16-byte word of its own row per lane).
template <int TNT>
__global__ __launch_bounds__(64) void g2bmm_kernel(BandParams p) {
    const int lane = threadIdx.x;
    const int l32 = lane & 31, hk = lane >> 5;
    int bx, by, bz;
    if (!band_position(p, bx, by, bz))
        return;
    const int b = bz / p.d, rho = bz - b * p.d;
    const int rows = rho < p.m ? (p.m - rho + p.d - 1) / p.d : 0; // rows of this class
    const int i0 = by * 32;
    if (i0 >= rows)
        return;
    // first column tile that can touch the band of rows i0 .. i0 + 31
    const int rfirst = i0 - p.w;
    const int r0 = rfirst + bx * (32 * TNT);
    if (r0 > i0 + 31 + p.w)
        return;
    const int ia = min(i0 + l32, rows - 1);
    const float *ap = p.A + ((size_t)b * p.m + rho + (size_t)ia * p.d) * p.k;
    const float *bp[TNT];
    bool rok[TNT], tile_on[TNT]; // tile_on: same for every lane
#pragma unroll
    for (int t = 0; t < TNT; ++t) {
        const int rb = r0 + t * 32 + l32;
        tile_on[t] = r0 + t * 32 <= i0 + 31 + p.w && r0 + t * 32 + 31 >= 0 && r0 + t * 32 < rows;
        rok[t] = tile_on[t] && rb >= 0 && rb < rows;
        bp[t] = p.B + ((size_t)b * p.m + rho + (size_t)(rok[t] ? rb : 0) * p.d) * p.k;
    }
    const bool vec = p.k % 8 == 0 && ((((uintptr_t)p.A) | ((uintptr_t)p.B)) & 15) == 0;
    floatx16 acc[TNT];
#pragma unroll
    for (int t = 0; t < TNT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[t][r] = 0.f;
    // U steps of 8 k values per trip: every load of a trip is issued before its first MFMA
    auto trip = [&](int k0, auto ucount) {
        constexpr int U = decltype(ucount)::value;
        float a[U][4], bv[U][TNT][4];
        if (vec) {
            // operand by operand: the U loads of one operand walk the same cache lines
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float4 va = *reinterpret_cast<const float4 *>(ap + k0 + u * 8 + hk * 4);
                a[u][0] = va.x, a[u][1] = va.y, a[u][2] = va.z, a[u][3] = va.w;
            }
#pragma unroll
            for (int t = 0; t < TNT; ++t)
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const float4 vb =
                        rok[t] ? *reinterpret_cast<const float4 *>(bp[t] + k0 + u * 8 + hk * 4)
                               : make_float4(0.f, 0.f, 0.f, 0.f);
                    bv[u][t][0] = vb.x, bv[u][t][1] = vb.y, bv[u][t][2] = vb.z, bv[u][t][3] = vb.w;
                }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kk = k0 + u * 8 + hk * 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    a[u][j] = kk + j < p.k ? ap[kk + j] : 0.f;
#pragma unroll
                    for (int t = 0; t < TNT; ++t)
                        bv[u][t][j] = (rok[t] && kk + j < p.k) ? bp[t][kk + j] : 0.f;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < TNT; ++t) {
            if (!tile_on[t])
                continue;
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][j], bv[u][t][j], acc[t], 0, 0,
                                                                   0);
        }
    };
    {
        int k0 = 0;
        if (TNT == 1)
            for (; k0 + 64 <= p.k; k0 += 64)
                trip(k0, std::integral_constant<int, 8>{});
        for (; k0 + 32 <= p.k; k0 += 32)
            trip(k0, std::integral_constant<int, 4>{});
        for (; k0 < p.k; k0 += 8)
            trip(k0, std::integral_constant<int, 1>{});
    }
    // register r: row i0 + (r/4)*8 + hk*4 + r%4, column r0 + 32 t + l32 -> band column j
    const int band = 2 * p.w + 1;
#pragma unroll
    for (int t = 0; t < TNT; ++t) {
        if (r0 + t * 32 > i0 + 31 + p.w)
            continue;
        const int rb = r0 + t * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int il = i0 + (r / 4) * 8 + hk * 4 + (r % 4);
            const int j = rb - il + p.w;
            if (il < rows && j >= 0 && j < band)
                p.C[((size_t)b * p.m + rho + (size_t)il * p.d) * band + j] = acc[t][r]; // 0 when !rok
        }
    }
}

struct __attribute__((packed, aligned(4))) Float4U {
    float x, y, z, w;
};

// ---- staged forms -------------------------------------------------------------------
// Both operands of G2BMM and the band operand of GBMML are contiguous along K, and the matrix
// core wants lane l of a half-wave to hold row l. Loaded that way (every lane a 16-byte word
// of its own row) one load instruction touches 32 cache lines. Here a wave reads a 32 x 32
// tile as consecutive 16-byte words, eight lanes to a row (8 lines per instruction), parks it
// in an LDS tile of its own (no workgroup barrier: the waves of a workgroup are independent)
// and reads it back in operand order: MFMA step j of a chunk takes k = hk * 16 + j.
constexpr int kKC = 32, kLD = kKC + 4, kTile = 32 * kLD;
constexpr int kWavesPerBlock = 4; // independent waves, grouped so that a CU holds more of them

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// operand order: row l32 of the parked tile, floats hk * 16 .. hk * 16 + 15
__device__ __forceinline__ void read_parked(const float *tile, int l32, int hk, float (&v)[16]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 f = *reinterpret_cast<const float4 *>(tile + l32 * kLD + hk * 16 + 4 * q);
        v[4 * q] = f.x, v[4 * q + 1] = f.y, v[4 * q + 2] = f.z, v[4 * q + 3] = f.w;
    }
}

// Addresses are 32-bit byte offsets into buffer resources based at the batch entry (one batch
// entry of every tensor stays under 2 GiB, checked on the host); an access that must not
// happen gets the offset kOob, which the range check turns into a zero (loads) or drops
// (stores). That keeps 64-bit arithmetic and branches out of the prologue and epilogue,
// which at k = 64 are as long as the MFMA work of a tile.
__device__ __forceinline__ void store_f32(float v, __amdgpu_buffer_rsrc_t r, unsigned off) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, off, 0, 0);
}

// k a multiple of 32, operands 16-byte aligned
__global__ __launch_bounds__(64 * kWavesPerBlock) void g2bmm_staged_kernel(BandParams p) {
    __shared__ __attribute__((aligned(16))) float lds_all[kWavesPerBlock * kTile];
    float *lds = lds_all + (threadIdx.x >> 6) * kTile;
    const int lane = threadIdx.x & 63;
    const int l32 = lane & 31, hk = lane >> 5;
    int bx, by, bz;
    if (!band_position(p, bx, by, bz))
        return;
    const int b = (int)fd_div((unsigned)bz, p.fd_d), rho = bz - b * p.d;
    const int rows = rho < p.m ? (p.m - rho + p.d - 1) / p.d : 0;
    const int i0 = by * 32;
    if (i0 >= rows)
        return;
    const int r0 = i0 - p.w + bx * 32;
    if (r0 > i0 + 31 + p.w)
        return;
    const int band = 2 * p.w + 1;
    const bool tile_on = r0 + 31 >= 0 && r0 < rows; // same for every lane
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A + (size_t)b * p.m * p.k);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B + (size_t)b * p.m * p.k);
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.C + (size_t)b * p.m * band);
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r)
        acc[r] = 0.f;
    if (tile_on) {
        // word q * 64 + lane of a tile: row q * 8 + lane / 8, floats 4 * (lane % 8) ..
        const int prow = lane >> 3, pc = lane & 7;
        unsigned voff[2][4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int row = q * 8 + prow;
            const int ia = min(i0 + row, rows - 1);
            voff[0][q] = ((unsigned)(rho + ia * p.d) * (unsigned)p.k + pc * 4) * 4u;
            const int rr = r0 + row;
            voff[1][q] = rr >= 0 && rr < rows
                             ? ((unsigned)(rho + rr * p.d) * (unsigned)p.k + pc * 4) * 4u
                             : kOob;
        }
        uintx4 stage[2][4];
        float a[16], bv[16];
        auto load = [&](int chunk) __attribute__((always_inline)) {
            const unsigned so = (unsigned)(chunk * kKC) * 4u;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                stage[0][q] = __builtin_amdgcn_raw_buffer_load_b128(ra, voff[0][q], so, 0);
                stage[1][q] = __builtin_amdgcn_raw_buffer_load_b128(rb, voff[1][q], so, 0);
            }
        };
        // the two operand tiles go through the wave's one LDS tile one after the other (a
        // small LDS footprint keeps many waves on a CU, which hides the load latency)
        auto park = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int o = 0; o < 2; ++o) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<uintx4 *>(lds + (q * 8 + prow) * kLD + pc * 4) = stage[o][q];
                wave_lds_fence();
                if (o == 0)
                    read_parked(lds, l32, hk, a);
                else
                    read_parked(lds, l32, hk, bv);
                wave_lds_fence();
            }
        };
        auto mma = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 16; ++j)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv[j], acc, 0, 0, 0);
        };
        const int nchunk = p.k / kKC;
        load(0);
        park();
        for (int chunk = 1; chunk < nchunk; ++chunk) {
            load(chunk);
            mma();
            park();
        }
        mma();
    }
    // register r: row il = i0 + hk*4 + ro(r), ro(r) = (r/4)*8 + r%4; column r0 + l32 is band
    // column j = r0 + l32 - il + w. Both move linearly with ro: offset0 + ro * (d*band - 1).
    // (A tile outside the rows of the class still stores its zeros.)
    const int il0 = i0 + hk * 4;
    const int j0 = r0 + l32 - il0 + p.w;
    const unsigned off0 = (unsigned)((rho + il0 * p.d) * band + j0) * 4u;
    const unsigned step = (unsigned)(p.d * band - 1) * 4u;
    const int rows_left = rows - il0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int ro = (r / 4) * 8 + (r % 4);
        const bool ok = ro < rows_left && (unsigned)(j0 - ro) < (unsigned)band;
        store_f32(acc[r], rc, ok ? off0 + (unsigned)ro * step : kOob);
    }
}

// The band operand's rows are 2w+1 floats, so its words are only 4-byte aligned; a chunk of
// 32 class rows is, for output row i', the 32 band columns from rc - i' + w on. Chunks in
// which every word of every row lies inside the band and the class take the fast path (one
// 16-byte load per word, no masks); the few at the ends of the K axis load float by float.
// SHARE: the waves of a workgroup take the K chunks of one tile in turn and add their partial
// tiles in LDS in wave order (for launches with too few tiles to keep the SIMDs busy).
template <int TN, bool SHARE>
__global__ __launch_bounds__(64 * kWavesPerBlock) void gbmml_staged_kernel(BandParams p) {
    constexpr int kPart = SHARE ? kWavesPerBlock * 32 * 32 * TN : 0;
    __shared__ __attribute__((aligned(16)))
    float lds_all[kPart > kWavesPerBlock * kTile ? kPart : kWavesPerBlock * kTile];
    const int wave = threadIdx.x >> 6;
    float *lds = lds_all + wave * kTile;
    const int lane = threadIdx.x & 63;
    const int l32 = lane & 31, hk = lane >> 5;
    int bx, by, bz;
    if (!band_position(p, bx, by, bz, !SHARE))
        return;
    const int b = (int)fd_div((unsigned)bz, p.fd_d), rho = bz - b * p.d;
    const int rows = rho < p.m ? (p.m - rho + p.d - 1) / p.d : 0;
    const int i0 = by * 32;
    if (i0 >= rows)
        return;
    const int n0 = bx * (32 * TN);
    const int band = 2 * p.w + 1;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(p.A + (size_t)b * p.m * band);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(p.B + (size_t)b * p.m * p.n);
    const __amdgpu_buffer_rsrc_t rc_out = make_rsrc(p.C + (size_t)b * p.m * p.n);
    bool nok[TN];
    unsigned boff[TN]; // class row 0, this lane's column
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
        nok[tn] = n0 + tn * 32 + l32 < p.n;
        boff[tn] = nok[tn] ? ((unsigned)rho * (unsigned)p.n + n0 + tn * 32 + l32) * 4u : kOob;
    }
    const unsigned brow = (unsigned)(p.d * p.n) * 4u; // bytes between class rows of B
    floatx16 acc[TN];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc[tn][r] = 0.f;
    const int klo = max(i0 - p.w, 0), khi = min(i0 + 31 + p.w, rows - 1);
    const int prow = lane >> 3, pc = lane & 7;
    // the four rows this lane stages: byte offset of band column 0, and jj - rc of its word
    unsigned aoff[4];
    int jbase[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int ia = min(i0 + q * 8 + prow, rows - 1);
        aoff[q] = (unsigned)(rho + ia * p.d) * (unsigned)band * 4u;
        jbase[q] = p.w - ia + pc * 4;
    }
    uintx4 stage[4];
    float a[16], bv[TN][16];
    auto load = [&](int rc, auto fast_tag) __attribute__((always_inline)) {
        constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int jj = rc + jbase[q]; // band column of this word's first float
            const int kk = rc + pc * 4;   // its class row
            if (FAST) {
                stage[q] = __builtin_amdgcn_raw_buffer_load_b128(ra, aoff[q] + (unsigned)jj * 4u, 0, 0);
            } else {
                unsigned e[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool ok = (unsigned)(jj + x) < (unsigned)band && kk + x <= khi;
                    e[x] = __builtin_amdgcn_raw_buffer_load_b32(
                        ra, ok ? aoff[q] + (unsigned)(jj + x) * 4u : kOob, 0, 0);
                }
                stage[q] = uintx4{e[0], e[1], e[2], e[3]};
            }
        }
        const unsigned so = (unsigned)(rc + hk * 16) * brow; // this half-wave's first class row
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const bool rin = FAST || rc + hk * 16 + j <= khi;
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                bv[tn][j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
                    rb, rin ? boff[tn] + so + (unsigned)j * brow : kOob, 0, 0));
        }
    };
    for (int rc = klo + (SHARE ? wave * kKC : 0); rc <= khi;
         rc += SHARE ? kWavesPerBlock * kKC : kKC) {
        // every row i0 .. i0+31 has band columns rc - i + w .. rc + 31 - i + w inside [0, band)
        const bool fast = rc >= i0 + 31 - p.w && rc + 31 <= i0 + p.w && rc + 31 <= khi;
        if (fast)
            load(rc, std::true_type{});
        else
            load(rc, std::false_type{});
#pragma unroll
        for (int q = 0; q < 4; ++q)
            *reinterpret_cast<uintx4 *>(lds + (q * 8 + prow) * kLD + pc * 4) = stage[q];
        wave_lds_fence();
        read_parked(lds, l32, hk, a);
        wave_lds_fence();
#pragma unroll
        for (int j = 0; j < 16; ++j)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
                acc[tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], bv[tn][j], acc[tn], 0, 0, 0);
    }
    if (!SHARE) {
        const int il0 = i0 + hk * 4;
        const int rows_left = rows - il0;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int ro = (r / 4) * 8 + (r % 4);
#pragma unroll
            for (int tn = 0; tn < TN; ++tn) {
                const unsigned off =
                    ((unsigned)(rho + (il0 + ro) * p.d) * (unsigned)p.n + n0 + tn * 32 + l32) * 4u;
                store_f32(acc[tn][r], rc_out, ro < rows_left && nok[tn] ? off : kOob);
            }
        }
        return;
    }
    constexpr int TW = 32 * TN;
    __syncthreads(); // every wave is done with its staging tile
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int r = 0; r < 16; ++r)
            lds_all[(wave * 32 + (r / 4) * 8 + hk * 4 + (r % 4)) * TW + tn * 32 + l32] = acc[tn][r];
    __syncthreads();
    for (int e = threadIdx.x; e < 32 * TW; e += 64 * kWavesPerBlock) {
        const int row = e / TW, col = e - row * TW;
        float v = lds_all[e];
#pragma unroll
        for (int w = 1; w < kWavesPerBlock; ++w)
            v += lds_all[w * 32 * TW + e];
        const bool ok = i0 + row < rows && n0 + col < p.n;
        store_f32(v, rc_out,
                  ok ? ((unsigned)(rho + (i0 + row) * p.d) * (unsigned)p.n + n0 + col) * 4u : kOob);
    }
}

// *empty: no batch entries or no rows, nothing to compute (pointers are not looked at).
int check_band(const float *A, const float *B, float *C, int bs, int m, int x, int w, int d,
               const char *what, bool *empty) {
    *empty = false;
    if (bs < 0 || m < 0 || x <= 0 || w < 0 || d <= 0)
        return set_error(PET_HIP_ERR_INVALID, "%s: bad shape bs=%d m=%d %d w=%d d=%d", what, bs, m,
                         x, w, d);
    if (bs == 0 || m == 0) {
        *empty = true;
        return PET_HIP_OK;
    }
    if (!A || !B || !C)
        return set_error(PET_HIP_ERR_INVALID, "%s: null operand", what);
    const long long band = 2ll * w + 1;
    if ((long long)bs * m * band >= (1ll << 31) || (long long)bs * m * x >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "%s: tensors of 2^31 elements or more", what);
    if ((long long)bs * d > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "%s: batch * dilation = %lld", what,
                         (long long)bs * d);
    return PET_HIP_OK;
}

// logical grid of gx * gy * gz waves, wpb of them to a workgroup
int band_grid(BandParams &p, int gx, int gy, int gz, int wpb, const char *what) {
    const long long total = (long long)gx * gy * gz;
    if (total <= 0 || total > (1ll << 30))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "%s: %lld tiles", what, total);
    p.gx = gx;
    p.gy = gy;
    p.fd_gx = make_fastdiv((unsigned)gx);
    p.fd_gy = make_fastdiv((unsigned)gy);
    p.fd_d = make_fastdiv((unsigned)p.d);
    p.total = (int)total;
    p.per_xcd = (int)(((total + wpb - 1) / wpb + 7) / 8);
    return PET_HIP_OK;
}

} // namespace

extern "C" {

int pet_hip_g2bmm_f32(const float *A, const float *B, float *C, int bs, int m, int k, int width,
                      int dilation, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    bool empty;
    if (int rc = check_band(A, B, C, bs, m, k, width, dilation, "g2bmm", &empty))
        return rc;
    if (empty)
        return PET_HIP_OK;
    BandParams p{A, B, C, bs, m, k, width, dilation, 0, 0, 0};
    p.mc = (m + dilation - 1) / dilation;
    // tiles from column i0 - w to i0 + 31 + w
    p.rtiles = (2 * width + 32 + 31) / 32;
    const unsigned iblocks = (unsigned)((p.mc + 31) / 32);
    if (iblocks > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "g2bmm: %d rows", m);
    const bool staged = k % kKC == 0 && ((((uintptr_t)A) | ((uintptr_t)B)) & 15) == 0 &&
                        (long long)m * k * 4 < (1ll << 31) &&
                        (long long)m * (2 * width + 1) * 4 < (1ll << 31);
    // column tiles per wave
    const int tpw = staged ? 1 : (p.rtiles >= 4 ? 4 : 1);
    const int wpb = staged ? kWavesPerBlock : 1;
    if (int rc = band_grid(p, (p.rtiles + tpw - 1) / tpw, (int)iblocks, bs * dilation, wpb,
                           "g2bmm"))
        return rc;
    const dim3 grid(8u * (unsigned)p.per_xcd);
    hipStream_t st = as_stream(stream);
    if (staged)
        hipLaunchKernelGGL(g2bmm_staged_kernel, grid, dim3(64 * wpb), 0, st, p);
    else if (tpw == 4)
        hipLaunchKernelGGL(g2bmm_kernel<4>, grid, dim3(64), 0, st, p);
    else
        hipLaunchKernelGGL(g2bmm_kernel<1>, grid, dim3(64), 0, st, p);
    return check_launch("g2bmm_kernel");
}

int pet_hip_gbmml_f32(const float *A, const float *B, float *C, int bs, int m, int width, int n,
                      int dilation, pet_hip_stream_t stream) {
    PET_REQUIRE_INIT();
    bool empty;
    if (int rc = check_band(A, B, C, bs, m, n, width, dilation, "gbmml", &empty))
        return rc;
    if (empty)
        return PET_HIP_OK;
    BandParams p{A, B, C, bs, m, 0, width, dilation, n, 0, 0};
    p.mc = (m + dilation - 1) / dilation;
    const unsigned iblocks = (unsigned)((p.mc + 31) / 32);
    if (iblocks > 65535)
        return set_error(PET_HIP_ERR_UNSUPPORTED, "gbmml: %d rows", m);
    if ((long long)m * (2 * width + 1) * 4 >= (1ll << 31) || (long long)m * n * 4 >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED, "gbmml: a batch entry of 2 GiB or more");
    // 64-column tiles, a tile per wave, when that gives the SIMDs a few waves each; else
    // 32-column tiles, or the waves of a workgroup sharing a tile's K axis
    const long long tiles64 = (long long)((n + 63) / 64) * iblocks * bs * dilation;
    const int tn = n > 32 && tiles64 >= 4096 ? 2 : 1;
    const long long tiles = (long long)((n + 32 * tn - 1) / (32 * tn)) * iblocks * bs * dilation;
    const bool share = tiles < 4096 && width >= 64;
    if (int rc = band_grid(p, (n + 32 * tn - 1) / (32 * tn), (int)iblocks, bs * dilation,
                           share ? 1 : kWavesPerBlock, "gbmml"))
        return rc;
    const dim3 grid(8u * (unsigned)p.per_xcd), block(64 * kWavesPerBlock);
    hipStream_t st = as_stream(stream);
    if (tn == 2) { // never shared: 64-column tiles are chosen only when there are many
        hipLaunchKernelGGL((gbmml_staged_kernel<2, false>), grid, block, 0, st, p);
    } else {
        if (share)
            hipLaunchKernelGGL((gbmml_staged_kernel<1, true>), grid, block, 0, st, p);
        else
            hipLaunchKernelGGL((gbmml_staged_kernel<1, false>), grid, block, 0, st, p);
    }
    return check_launch("gbmml_staged_kernel");
}

} // extern "C"
