// View-copy engine: canonicalisation, kernel selection and the two kernels
// (direct and LDS-tiled) behind every layout operator.
#include "view.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace pet {

// Division by a run-time invariant through multiply-high; valid for
// dividends below 2^31.
struct FastDiv {
    unsigned d, mul, shift;
};

static FastDiv make_fastdiv(unsigned d) {
    FastDiv f;
    f.d = d;
    if (d <= 1) {
        f.mul = 0;
        f.shift = 0;
        return f;
    }
    unsigned l = 0;
    while ((1ull << l) < d)
        ++l;
    unsigned p = 31 + l;
    unsigned long long m = ((1ull << p) + d - 1) / d;
    f.mul = (unsigned)m;
    f.shift = p - 32;
    return f;
}

__device__ __forceinline__ unsigned fd_div(unsigned n, const FastDiv &f) {
    return f.d == 1 ? n : (__umulhi(n, f.mul) >> f.shift);
}

struct DirectParams {
    int rank;          // canonical rank, innermost last
    FastDiv ext[PET_HIP_MAX_RANK];
    FastDiv m[PET_HIP_MAX_RANK];
    int has_div[PET_HIP_MAX_RANK];
    int lo[PET_HIP_MAX_RANK], hi[PET_HIP_MAX_RANK];
    long long os[PET_HIP_MAX_RANK], sq[PET_HIP_MAX_RANK], sr[PET_HIP_MAX_RANK];
    long long ibase, obase;
    unsigned total; // number of work items (elements / VEC)
    int inner_contig; // the innermost dim is contiguous in the input and has no div level
};

typedef float vf4 __attribute__((ext_vector_type(4)));
// the same four floats at 4-byte alignment: the hardware takes a 16-byte load at any
// dword address (the compiler itself emits one for this type)
typedef float vf4u __attribute__((ext_vector_type(4), aligned(4)));

// Streaming (non-temporal) accesses for tensors too large to stay in cache.
template <bool NT>
__device__ __forceinline__ vf4 ld4(const float *p) {
    const vf4 *q = reinterpret_cast<const vf4 *>(p);
    return NT ? __builtin_nontemporal_load(q) : *q;
}
template <bool NT>
__device__ __forceinline__ void st4(float *p, vf4 v) {
    vf4 *q = reinterpret_cast<vf4 *>(p);
    if (NT)
        __builtin_nontemporal_store(v, q);
    else
        *q = v;
}

// One work item = VEC consecutive elements of the innermost iteration dim.
// With VEC == 4 the host has checked that the four elements are contiguous and
// 16-byte aligned on both sides and share one validity result. A thread takes
// UN items 256 apart and issues all its loads before its stores, so UN 16-byte
// requests per lane are in flight.
template <int VEC, int UN, bool NT>
__global__ __launch_bounds__(256) void view_direct_kernel(const float *__restrict__ x,
                                                          float *__restrict__ y,
                                                          DirectParams p) {
    const unsigned base = blockIdx.x * (256u * UN) + threadIdx.x;
    long long io[UN], oo[UN];
    bool ok[UN], live[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const unsigned t = base + u * 256u;
        live[u] = t < p.total;
        unsigned rem = live[u] ? t : 0u;
        io[u] = p.ibase;
        oo[u] = p.obase;
        ok[u] = live[u];
#pragma unroll
        for (int d = PET_HIP_MAX_RANK - 1; d >= 0; --d) {
            if (d < p.rank) {
                unsigned q = fd_div(rem, p.ext[d]);
                unsigned idx = rem - q * p.ext[d].d;
                rem = q;
                if (d == p.rank - 1)
                    idx *= VEC;
                oo[u] += (long long)idx * p.os[d];
                unsigned r = idx;
                if (p.has_div[d]) {
                    unsigned qq = fd_div(idx, p.m[d]);
                    r = idx - qq * p.m[d].d;
                    io[u] += (long long)qq * p.sq[d];
                }
                io[u] += (long long)r * p.sr[d];
                ok[u] = ok[u] && ((int)r >= p.lo[d]) && ((int)r < p.hi[d]);
            }
        }
    }
    if (VEC == 4) {
        vf4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            v[u] = (vf4){0.f, 0.f, 0.f, 0.f};
            if (ok[u])
                v[u] = ld4<NT>(x + io[u]);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (live[u])
                st4<NT>(y + oo[u], v[u]);
    } else {
        float v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u)
            v[u] = ok[u] ? x[io[u]] : 0.f;
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (live[u])
                y[oo[u]] = v[u];
    }
}

// Index of one element of the iteration space -> input offset and validity,
// split into the innermost dim and the rest so that neighbours along a row reuse
// the outer part. 32-bit wrap-around arithmetic: both buffers hold fewer than
// 2^31 elements, so the offset of every valid element is exact modulo 2^32.
// Row index (all dims but the innermost, flattened) -> input offset of the row's
// element 0 and whether the row lies inside every outer window.
__device__ __forceinline__ void decode_row(const DirectParams &p, unsigned e, unsigned &io,
                                           bool &ok) {
    io = (unsigned)p.ibase;
    const int L = p.rank - 1;
#pragma unroll
    for (int d = PET_HIP_MAX_RANK - 2; d >= 0; --d) {
        if (d < L) {
            unsigned q = fd_div(e, p.ext[d]);
            unsigned r = e - q * p.ext[d].d;
            e = q;
            if (p.has_div[d]) {
                unsigned qq = fd_div(r, p.m[d]);
                r -= qq * p.m[d].d;
                io += qq * (unsigned)p.sq[d];
            }
            io += r * (unsigned)p.sr[d];
            ok = ok && ((int)r >= p.lo[d]) && ((int)r < p.hi[d]);
        }
    }
}

__device__ __forceinline__ void decode_outer(const DirectParams &p, unsigned e, unsigned &inner,
                                             unsigned &io, bool &ok) {
    const int L = p.rank - 1;
    unsigned q = fd_div(e, p.ext[L]);
    inner = e - q * p.ext[L].d;
    decode_row(p, q, io, ok);
}

__device__ __forceinline__ void eval_inner(const DirectParams &p, unsigned r, unsigned &io,
                                           bool &ok) {
    const int L = p.rank - 1;
    if (p.has_div[L]) {
        unsigned qq = fd_div(r, p.m[L]);
        r -= qq * p.m[L].d;
        io += qq * (unsigned)p.sq[L];
    }
    io += r * (unsigned)p.sr[L];
    ok = ok && ((int)r >= p.lo[L]) && ((int)r < p.hi[L]);
}

// Dense, 16-byte aligned output but an input side that cannot be vectorised (an
// innermost extent that is not a multiple of 4, a window that cuts through
// it): a thread gathers 4 consecutive output elements one by one and stores
// them as one 16-byte word. p.total counts the 4-element groups; the output
// offset of group t is obase + 4t.
template <bool NT>
__global__ __launch_bounds__(256) void view_gather4_kernel(const float *__restrict__ x,
                                                           float *__restrict__ y,
                                                           DirectParams p) {
    constexpr int UN = 4;
    const unsigned base = blockIdx.x * (256u * UN) + threadIdx.x;
    const unsigned ext_inner = p.ext[p.rank - 1].d;
    float v[UN][4];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const unsigned t = base + u * 256u;
        const bool live = t < p.total;
        const unsigned e0 = live ? t * 4u : 0u;
        unsigned inner, io_outer;
        bool ok_outer = live;
        decode_outer(p, e0, inner, io_outer, ok_outer);
        // the common case: all four inside one row and inside its window, the row
        // contiguous in the input -> one 16-byte load at whatever dword alignment
        const int L = p.rank - 1;
        if (p.inner_contig && ok_outer && inner + 3 < ext_inner && (int)inner >= p.lo[L] &&
            (int)inner + 3 < p.hi[L]) {
            const vf4u *src = reinterpret_cast<const vf4u *>(x + (io_outer + inner * (unsigned)p.sr[L]));
            const vf4u w = NT ? __builtin_nontemporal_load(src) : *src;
            v[u][0] = w.x;
            v[u][1] = w.y;
            v[u][2] = w.z;
            v[u][3] = w.w;
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (j > 0 && ++inner == ext_inner) { // next row: decode afresh
                ok_outer = live;
                decode_outer(p, e0 + j, inner, io_outer, ok_outer);
            }
            unsigned io = io_outer;
            bool ok = ok_outer;
            eval_inner(p, inner, io, ok);
            v[u][j] = 0.f;
            if (ok)
                v[u][j] = NT ? __builtin_nontemporal_load(x + io) : x[io];
        }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const unsigned t = base + u * 256u;
        if (t < p.total)
            st4<NT>(y + p.obase + 4ll * t, (vf4){v[u][0], v[u][1], v[u][2], v[u][3]});
    }
}

// Dense, 16-byte aligned output whose rows are contiguous pieces of the input at
// any dword alignment (a cropped or zero-padded innermost dim, an odd row length):
// a workgroup produces ROWSTAGE_TILE consecutive output elements in LDS and
// stores them as aligned 16-byte words. The rows that meet the tile are fetched
// as the ALIGNED 16-byte input words that cover them, one word per work item,
// and scattered element-wise into the LDS tile at their output position, so
// that both global sides move whole aligned words however the two row lengths
// relate. An aligned word that holds one valid element lies inside that
// element's page, so the up to three neighbours it brings along are always
// readable; they are dropped. Elements outside the windows keep the zeros the
// tile is cleared to (only views that have such elements clear it).
constexpr unsigned ROWSTAGE_TILE = 4096;
struct RowStageParams {
    FastDiv cpr;        // upper bound of the aligned input words one row needs inside a tile
    int zero;           // some window is narrower than its dim
    unsigned total;     // output elements
};

template <bool NT>
__global__ __launch_bounds__(256) void view_rowstage_kernel(const float *__restrict__ x,
                                                            float *__restrict__ y,
                                                            DirectParams p, RowStageParams rs) {
    constexpr unsigned T = ROWSTAGE_TILE;
    constexpr int UN = 4;
    __shared__ __attribute__((aligned(16))) float tile[T];
    const unsigned tid = threadIdx.x;
    const unsigned E0 = blockIdx.x * T;
    const unsigned E1 = min(E0 + T, rs.total);
    const int L = p.rank - 1;
    const unsigned ext_inner = p.ext[L].d;
    const int lo = p.lo[L], hi = p.hi[L];
    const unsigned r0 = fd_div(E0, p.ext[L]);
    const unsigned r1 = fd_div(E1 - 1u, p.ext[L]);
    const unsigned items = (r1 - r0 + 1u) * rs.cpr.d;
    if (rs.zero) {
#pragma unroll
        for (unsigned u = 0; u < T / 1024u; ++u)
            *reinterpret_cast<vf4 *>(&tile[(u * 256u + tid) * 4u]) = (vf4){0.f, 0.f, 0.f, 0.f};
        __syncthreads();
    }
    for (unsigned it0 = 0; it0 < items; it0 += 256u * UN) {
        vf4 w[UN];
        int first[UN], a[UN], b[UN], rel[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const unsigned it = it0 + u * 256u + tid;
            a[u] = 0;
            b[u] = 0;
            first[u] = 0;
            rel[u] = 0;
            w[u] = (vf4){0.f, 0.f, 0.f, 0.f};
            if (it < items) {
                const unsigned rl = fd_div(it, rs.cpr);
                const unsigned ch = it - rl * rs.cpr.d;
                const unsigned row = r0 + rl;
                unsigned io_row;
                bool ok = true;
                decode_row(p, row, io_row, ok);
                const unsigned row_start = row * ext_inner;
                // the part of this row inside the tile and the window, as inner indices
                const int aa = max((int)(E0 > row_start ? E0 - row_start : 0u), lo);
                const int bb = min((int)(min(E1, row_start + ext_inner) - row_start), hi);
                if (ok && aa < bb) {
                    const unsigned g = io_row + (unsigned)aa; // input offset of inner index aa
                    const unsigned mis = g & 3u;
                    const int ii = aa - (int)mis + 4 * (int)ch;
                    if (ii < bb) {
                        w[u] = ld4<NT>(x + ((g - mis) + 4u * ch));
                        a[u] = aa;
                        b[u] = bb;
                        first[u] = ii;
                        rel[u] = (int)(row_start - E0); // wraps to the negative offset of a row that began before the tile
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = first[u] + j;
                if (i >= a[u] && i < b[u])
                    tile[rel[u] + i] = w[u][j];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (unsigned u = 0; u < T / 1024u; ++u) {
        const unsigned idx = (u * 256u + tid) * 4u;
        if (E0 + idx < E1)
            st4<NT>(y + p.obase + (long long)(E0 + idx),
                    *reinterpret_cast<const vf4 *>(&tile[idx]));
    }
}

// Interleave kernels for the space-to-batch family: a dim of extent E (2 or 4)
// that is innermost on one side sits next to the dim that is innermost on the
// other side. DEINT: the input holds (w, e) with e innermost and the output has
// w innermost with the planes e far apart (space-to-batch); otherwise the
// reverse (batch-to-space). 16-byte accesses on both sides, no LDS.
struct InterleaveParams {
    DirectParams dp;   // the iteration space without the E dim; innermost dim in units of 4
    long long e_stride; // stride of the E dim on the side where it is not innermost
};

// The 2-wide case moves whole cache lines on both sides: a lane handles one
// 16-byte word of the interleaved side and, with its neighbour (lane ^ 1),
// one word of each of the two planes; the pair swaps two floats each through a
// lane shuffle. p's last dim counts the interleaved row in 16-byte words.
template <bool DEINT, bool NT>
__global__ __launch_bounds__(256) void view_interleave2_kernel(const float *__restrict__ x,
                                                               float *__restrict__ y,
                                                               InterleaveParams ip) {
    const DirectParams &p = ip.dp;
    constexpr int UN = 4;
    const unsigned base = blockIdx.x * (256u * UN) + threadIdx.x;
    const bool odd = threadIdx.x & 1;
    unsigned io[UN], oo[UN];
    bool live[UN];
    vf4 a[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const unsigned t = base + u * 256u;
        live[u] = t < p.total; // the same for both lanes of a pair: total is even
        unsigned rem = live[u] ? t : 0u;
        io[u] = (unsigned)p.ibase;
        oo[u] = (unsigned)p.obase;
#pragma unroll
        for (int d = PET_HIP_MAX_RANK - 1; d >= 0; --d) {
            if (d < p.rank) {
                unsigned q = fd_div(rem, p.ext[d]);
                unsigned idx = rem - q * p.ext[d].d;
                rem = q;
                if (d == p.rank - 1) {
                    // word idx of the interleaved row <-> word idx/2 of plane idx%2
                    const unsigned planar = 4u * (idx >> 1) + (idx & 1) * (unsigned)ip.e_stride;
                    io[u] += DEINT ? 4u * idx : planar;
                    oo[u] += DEINT ? planar : 4u * idx;
                } else {
                    oo[u] += idx * (unsigned)p.os[d];
                    io[u] += idx * (unsigned)p.sr[d];
                }
            }
        }
        a[u] = (vf4){0.f, 0.f, 0.f, 0.f};
        if (live[u])
            a[u] = ld4<NT>(x + io[u]);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const vf4 v = a[u];
        vf4 o;
        if (DEINT) {
            // even lane keeps plane 0 (x, z) and wants the neighbour's; odd likewise for plane 1
            const float r0 = __shfl_xor(odd ? v.x : v.y, 1);
            const float r1 = __shfl_xor(odd ? v.z : v.w, 1);
            o = odd ? (vf4){r0, r1, v.y, v.w} : (vf4){v.x, v.z, r0, r1};
        } else {
            const float r0 = __shfl_xor(odd ? v.x : v.z, 1);
            const float r1 = __shfl_xor(odd ? v.y : v.w, 1);
            o = odd ? (vf4){r0, v.z, r1, v.w} : (vf4){v.x, r0, v.y, r1};
        }
        if (live[u])
            st4<NT>(y + oo[u], o);
    }
}

// The 4-wide case: a lane holds one 16-byte word (one position, four planes, or
// the reverse); the four lanes of a quad transpose their 4x4 block in three
// exchange rounds. p's last dim counts positions of the interleaved row.
template <bool DEINT, bool NT>
__global__ __launch_bounds__(256) void view_interleave4_kernel(const float *__restrict__ x,
                                                               float *__restrict__ y,
                                                               InterleaveParams ip) {
    const DirectParams &p = ip.dp;
    constexpr int UN = 4;
    const unsigned base = blockIdx.x * (256u * UN) + threadIdx.x;
    const unsigned q4 = threadIdx.x & 3;
    unsigned oo[UN];
    bool live[UN];
    vf4 a[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const unsigned t = base + u * 256u;
        live[u] = t < p.total; // the same for a whole quad: total is a multiple of 4
        unsigned rem = live[u] ? t : 0u;
        unsigned io = (unsigned)p.ibase;
        oo[u] = (unsigned)p.obase;
#pragma unroll
        for (int d = PET_HIP_MAX_RANK - 1; d >= 0; --d) {
            if (d < p.rank) {
                unsigned q = fd_div(rem, p.ext[d]);
                unsigned idx = rem - q * p.ext[d].d;
                rem = q;
                if (d == p.rank - 1) {
                    const unsigned planar = 4u * (idx >> 2) + (idx & 3) * (unsigned)ip.e_stride;
                    io += DEINT ? 4u * idx : planar;
                    oo[u] += DEINT ? planar : 4u * idx;
                } else {
                    oo[u] += idx * (unsigned)p.os[d];
                    io += idx * (unsigned)p.sr[d];
                }
            }
        }
        a[u] = (vf4){0.f, 0.f, 0.f, 0.f};
        if (live[u])
            a[u] = ld4<NT>(x + io);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const vf4 v = a[u];
        float o[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            // partner = q4 ^ r: it needs my element `partner`, I need its element q4
            const unsigned pr = q4 ^ r;
            const float send = pr == 0 ? v.x : pr == 1 ? v.y : pr == 2 ? v.z : v.w;
            const float recv = r == 0 ? send : __shfl_xor(send, r);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (r == 0)
                    o[j] = recv; // every slot is overwritten below except slot q4
                else
                    o[j] = pr == (unsigned)j ? recv : o[j];
        }
        if (live[u])
            st4<NT>(y + oo[u], (vf4){o[0], o[1], o[2], o[3]});
    }
}

// ---- LDS-tiled kernel --------------------------------------------------------
// Up to 4 tile dims with power-of-two tile extents. Elements are read in
// "input order" (tile dims sorted by input stride, so consecutive lanes read
// consecutive addresses), parked in LDS, and written in "output order" (sorted
// by output stride). Dims outside the tile are handled by the grid.
constexpr int kTileDims = 4;

struct TiledParams {
    int rank;
    // non-tile dims are decoded from blockIdx by the workgroup
    FastDiv gdiv[PET_HIP_MAX_RANK];   // product of tile counts of the dims inside d
    FastDiv ntiles[PET_HIP_MAX_RANK]; // number of tiles along d
    int is_tile[PET_HIP_MAX_RANK];
    int has_div[PET_HIP_MAX_RANK];
    FastDiv m[PET_HIP_MAX_RANK];
    int lo[PET_HIP_MAX_RANK], hi[PET_HIP_MAX_RANK];
    long long os[PET_HIP_MAX_RANK], sq[PET_HIP_MAX_RANK], sr[PET_HIP_MAX_RANK];
    long long ibase, obase;
    int ntd; // number of tile dims
    // tile dims in input order (ascending input stride)
    FastDiv in_gdiv[kTileDims], in_nt[kTileDims];
    int in_shift[kTileDims], in_ext[kTileDims];
    long long in_sr[kTileDims];
    // the same dims in output order (ascending output stride)
    FastDiv out_gdiv[kTileDims], out_nt[kTileDims];
    int out_shift[kTileDims], out_ext[kTileDims];
    long long out_os[kTileDims];
    int out_to_in_pos[kTileDims]; // bit offset of the dim in the input-order linear id
    int tile_elems;
};

// VIN / VOUT: the host has checked that four consecutive elements in input
// (output) order are contiguous, 16-byte aligned and valid together, so the
// global side moves 16 bytes per lane. Loads of a pass are all issued before the
// LDS writes (four requests per lane in flight).
template <bool VIN, bool VOUT, bool NT>
__global__ __launch_bounds__(256) void view_tiled_kernel(const float *__restrict__ x,
                                                         float *__restrict__ y,
                                                         TiledParams p) {
    extern __shared__ float lds[]; // tile_elems * 33 / 32 floats
    const unsigned wg = blockIdx.x;
    long long ibase = p.ibase, obase = p.obase;
    bool wg_ok = true;
#pragma unroll
    for (int d = 0; d < PET_HIP_MAX_RANK; ++d) {
        if (d < p.rank && !p.is_tile[d]) {
            unsigned q = fd_div(wg, p.gdiv[d]);
            unsigned idx = q - fd_div(q, p.ntiles[d]) * p.ntiles[d].d;
            unsigned r = idx;
            obase += (long long)idx * p.os[d];
            if (p.has_div[d]) {
                unsigned qq = fd_div(idx, p.m[d]);
                r = idx - qq * p.m[d].d;
                ibase += (long long)qq * p.sq[d];
            }
            ibase += (long long)r * p.sr[d];
            wg_ok = wg_ok && ((int)r >= p.lo[d]) && ((int)r < p.hi[d]);
        }
    }
    int org_in[kTileDims], org_out[kTileDims];
#pragma unroll
    for (int i = 0; i < kTileDims; ++i) {
        org_in[i] = org_out[i] = 0;
        if (i < p.ntd) {
            unsigned q = fd_div(wg, p.in_gdiv[i]);
            org_in[i] = (int)((q - fd_div(q, p.in_nt[i]) * p.in_nt[i].d) << p.in_shift[i]);
            q = fd_div(wg, p.out_gdiv[i]);
            org_out[i] = (int)((q - fd_div(q, p.out_nt[i]) * p.out_nt[i].d) << p.out_shift[i]);
        }
    }
    constexpr int UN = 4;
    // load phase: consecutive lanes walk the tile in input order
    {
        constexpr int W = VIN ? 4 : 1;
        const int items = p.tile_elems / W;
        for (int b = 0; b < items; b += 256 * UN) {
            vf4 v[UN];
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int t = b + u * 256 + (int)threadIdx.x;
                int remt = t * W;
                long long io = ibase;
                bool ok = wg_ok && t < items;
#pragma unroll
                for (int i = 0; i < kTileDims; ++i) {
                    if (i < p.ntd) {
                        int c = remt & ((1 << p.in_shift[i]) - 1);
                        remt >>= p.in_shift[i];
                        int idx = org_in[i] + c;
                        ok = ok && idx < p.in_ext[i];
                        io += (long long)idx * p.in_sr[i];
                    }
                }
                v[u] = (vf4){0.f, 0.f, 0.f, 0.f};
                if (ok) {
                    if (VIN)
                        v[u] = ld4<NT>(x + io);
                    else
                        v[u].x = NT ? __builtin_nontemporal_load(x + io) : x[io];
                }
            }
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const int t = b + u * 256 + (int)threadIdx.x;
                if (t < items) {
                    if (VIN) {
                        const int e = t * 4, pad = e >> 5; // 4 | 32: one pad for all four
                        lds[e + pad] = v[u].x;
                        lds[e + 1 + pad] = v[u].y;
                        lds[e + 2 + pad] = v[u].z;
                        lds[e + 3 + pad] = v[u].w;
                    } else {
                        lds[t + (t >> 5)] = v[u].x;
                    }
                }
            }
        }
    }
    __syncthreads();
    // store phase: consecutive lanes walk the tile in output order
    {
        constexpr int W = VOUT ? 4 : 1;
        const int items = p.tile_elems / W;
        for (int t = threadIdx.x; t < items; t += 256) {
            int remt = t * W;
            long long oo = obase;
            bool ok = true;
#pragma unroll
            for (int i = 0; i < kTileDims; ++i) {
                if (i < p.ntd) {
                    int c = remt & ((1 << p.out_shift[i]) - 1);
                    remt >>= p.out_shift[i];
                    int idx = org_out[i] + c;
                    ok = ok && idx < p.out_ext[i];
                    oo += (long long)idx * p.out_os[i];
                }
            }
            if (!ok)
                continue;
            float r[W];
#pragma unroll
            for (int j = 0; j < W; ++j) {
                int e = t * W + j, lin = 0;
#pragma unroll
                for (int i = 0; i < kTileDims; ++i) {
                    if (i < p.ntd) {
                        lin += (e & ((1 << p.out_shift[i]) - 1)) << p.out_to_in_pos[i];
                        e >>= p.out_shift[i];
                    }
                }
                r[j] = lds[lin + (lin >> 5)];
            }
            if (VOUT) {
                st4<NT>(y + oo, (vf4){r[0], r[W > 1 ? 1 : 0], r[W > 2 ? 2 : 0], r[W > 3 ? 3 : 0]});
            } else {
                if (NT)
                    __builtin_nontemporal_store(r[0], y + oo);
                else
                    y[oo] = r[0];
            }
        }
    }
}

// Tensors beyond this many elements (256 MiB in + out) cannot stay in the
// last-level cache between kernels: stream them with non-temporal accesses.
static inline bool stream_sized(long long total) {
    static const long long thr = getenv("PET_HIP_VIEW_NT")
                                     ? atoll(getenv("PET_HIP_VIEW_NT"))
                                     : (32ll << 20);
    return total >= thr;
}

template <bool VI, bool VO, bool NTF>
static void launch_tiled(dim3 grid, size_t lds_bytes, hipStream_t stream, const float *x, float *y,
                         const TiledParams &p) {
    // tiles beyond 64 KiB of LDS need the limit raised once per kernel
    static const bool raised = [] {
        return hipFuncSetAttribute(
                   reinterpret_cast<const void *>(&view_tiled_kernel<VI, VO, NTF>),
                   hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024) == hipSuccess;
    }();
    (void)raised;
    hipLaunchKernelGGL((view_tiled_kernel<VI, VO, NTF>), grid, dim3(256), lds_bytes, stream, x, y,
                       p);
}

static inline bool plain(const ViewDim &d) {
    return d.m >= d.ext && d.lo <= 0 && d.hi >= d.ext;
}

static int ceil_log2(int v) {
    int l = 0;
    while ((1 << l) < v)
        ++l;
    return l;
}

// Host-side bounds check of the whole index space: every valid read stays in
// [0, in_elems) and every write in [0, out_elems).
static bool view_in_bounds(const ViewDesc &v, long long in_elems, long long out_elems) {
    long long imin = v.ibase, imax = v.ibase, omin = v.obase, omax = v.obase;
    for (int i = 0; i < v.rank; ++i) {
        const ViewDim &d = v.d[i];
        if (d.ext <= 0)
            return false;
        long long oe = (long long)(d.ext - 1) * d.os;
        (oe < 0 ? omin : omax) += oe;
        // valid r range
        int m = d.m >= d.ext ? d.ext : d.m;
        int rlo = std::max(0, d.lo), rhi = std::min(m, d.hi) - 1;
        if (rhi < rlo)
            continue; // nothing valid along this dim: no read at all, but keep going
        long long a = (long long)rlo * d.sr, b = (long long)rhi * d.sr;
        imin += std::min(a, b);
        imax += std::max(a, b);
        if (d.m < d.ext) {
            long long qmax = (d.ext - 1) / d.m;
            long long e = qmax * d.sq;
            (e < 0 ? imin : imax) += e;
        }
    }
    if (omin < 0 || omax >= out_elems)
        return false;
    if (imin < 0 || imax >= in_elems)
        return false;
    return true;
}

int launch_view_copy(const float *x, float *y, ViewDesc v, long long in_elems,
                     long long out_elems, hipStream_t stream) {
    if (v.rank < 0 || v.rank > PET_HIP_MAX_RANK)
        return set_error(PET_HIP_ERR_INVALID, "view rank %d out of range", v.rank);
    long long total = 1;
    for (int i = 0; i < v.rank; ++i) {
        if (v.d[i].ext < 0)
            return set_error(PET_HIP_ERR_INVALID, "negative extent");
        total *= v.d[i].ext;
    }
    if (total == 0)
        return PET_HIP_OK; // empty tensor: nothing to do
    if (total >= (1ll << 31) || in_elems >= (1ll << 31) || out_elems >= (1ll << 31))
        return set_error(PET_HIP_ERR_UNSUPPORTED,
                         "layout ops are limited to tensors below 2^31 elements");
    if (!y)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    if (in_elems == 0) // padding around an empty tensor: nothing to read, all zeros
        return pet_hip_fill_f32(y, 0.f, (size_t)out_elems, (pet_hip_stream_t)stream);
    if (!x)
        return set_error(PET_HIP_ERR_INVALID, "null tensor pointer");
    // does any element read at all? (a dim whose window is empty zero-fills)
    bool any_valid = true;
    for (int i = 0; i < v.rank; ++i) {
        const ViewDim &d = v.d[i];
        int m = d.m >= d.ext ? d.ext : d.m;
        if (std::min(m, d.hi) <= std::max(0, d.lo))
            any_valid = false;
    }
    if (any_valid && !view_in_bounds(v, in_elems, out_elems))
        return set_error(PET_HIP_ERR_INVALID, "view reaches outside its buffers");

    // ---- canonicalise: drop unit dims, merge adjacent compatible dims
    ViewDesc c;
    c.rank = 0;
    c.ibase = v.ibase;
    c.obase = v.obase;
    for (int i = 0; i < v.rank; ++i) {
        ViewDim d = v.d[i];
        if (d.ext == 1) {
            // index 0: q = 0, r = 0
            if (!(d.lo <= 0 && d.hi > 0)) {
                // permanently invalid: keep it so the kernel zero-fills
                c.d[c.rank++] = d;
            }
            continue;
        }
        if (d.m >= d.ext) {
            d.m = d.ext;
            d.sq = 0;
            d.hi = std::min(d.hi, d.ext);
            d.lo = std::max(d.lo, 0);
        }
        if (c.rank > 0) {
            ViewDim &pdim = c.d[c.rank - 1];
            if (plain(pdim) && plain(d) && pdim.os == d.os * d.ext && pdim.sr == d.sr * d.ext &&
                (long long)pdim.ext * d.ext < (1ll << 31)) {
                pdim.ext *= d.ext;
                pdim.m = pdim.ext;
                pdim.hi = pdim.ext;
                pdim.os = d.os;
                pdim.sr = d.sr;
                continue;
            }
        }
        c.d[c.rank++] = d;
    }
    if (c.rank == 0) {
        c.rank = 1;
        c.d[0] = ViewDim{1, 1, 0, 1, 1, 0, 1};
    }

    const int L = c.rank - 1;
    const ViewDim &inner = c.d[L];
    bool inner_coalesced_out = inner.os == 1;
    bool inner_coalesced_in = plain(inner) ? inner.sr == 1 : (inner.sr == 1);

    // ---- interleave path: a 2- or 4-wide dim innermost on one side, adjacent to
    // the dim that is innermost on the other side (space-to-batch and its inverse)
    {
        const bool aligned = c.ibase % 4 == 0 && c.obase % 4 == 0 && (uintptr_t)x % 16 == 0 &&
                             (uintptr_t)y % 16 == 0;
        int kE = -1, kW = -1;
        bool deint = false;
        if (aligned && plain(inner) && inner.os == 1 && (inner.sr == 2 || inner.sr == 4) &&
            inner.ext % 4 == 0) {
            // output innermost = w; look for the E dim (input innermost)
            for (int i = 0; i < L; ++i)
                if (plain(c.d[i]) && c.d[i].sr == 1 && c.d[i].ext == inner.sr && c.d[i].os % 4 == 0)
                    kE = i;
            kW = L;
            deint = true;
        } else if (aligned && plain(inner) && inner.os == 1 && (inner.ext == 2 || inner.ext == 4) &&
                   inner.sr % 4 == 0) {
            // output innermost = the E dim; look for w (input innermost)
            for (int i = 0; i < L; ++i)
                if (plain(c.d[i]) && c.d[i].sr == 1 && c.d[i].os == inner.ext &&
                    c.d[i].ext % 4 == 0)
                    kW = i;
            kE = L;
        }
        bool ok = kE >= 0 && kW >= 0 && kE != kW;
        for (int i = 0; ok && i < c.rank; ++i) {
            if (i == kE || i == kW)
                continue;
            const ViewDim &d = c.d[i];
            if (!plain(d) || d.os % 4 || d.sr % 4)
                ok = false;
        }
        if (ok) {
            InterleaveParams ip;
            memset(&ip, 0, sizeof(ip));
            DirectParams &p = ip.dp;
            p.ibase = c.ibase;
            p.obase = c.obase;
            int r = 0;
            auto put = [&](const ViewDim &d, int ext) {
                p.ext[r] = make_fastdiv((unsigned)ext);
                p.os[r] = d.os;
                p.sr[r] = d.sr;
                ++r;
            };
            for (int i = 0; i < c.rank; ++i)
                if (i != kE && i != kW)
                    put(c.d[i], c.d[i].ext);
            const int E = c.d[kE].ext;
            // E == 2: the last dim counts 16-byte words of the interleaved row
            put(c.d[kW], E == 2 ? c.d[kW].ext / 2 : c.d[kW].ext);
            p.rank = r;
            ip.e_stride = deint ? c.d[kE].os : c.d[kE].sr;
            const long long items = total / 4;
            p.total = (unsigned)items;
            const bool nt = stream_sized(total);
            const unsigned per_wg = 256u * 4;
            const dim3 grid((unsigned)((items + per_wg - 1) / per_wg)), block(256);
            if (E == 2) {
                if (deint && nt)
                    hipLaunchKernelGGL((view_interleave2_kernel<true, true>), grid, block, 0,
                                       stream, x, y, ip);
                else if (deint)
                    hipLaunchKernelGGL((view_interleave2_kernel<true, false>), grid, block, 0,
                                       stream, x, y, ip);
                else if (nt)
                    hipLaunchKernelGGL((view_interleave2_kernel<false, true>), grid, block, 0,
                                       stream, x, y, ip);
                else
                    hipLaunchKernelGGL((view_interleave2_kernel<false, false>), grid, block, 0,
                                       stream, x, y, ip);
                return check_launch("view_interleave2_kernel");
            }
            if (deint && nt)
                hipLaunchKernelGGL((view_interleave4_kernel<true, true>), grid, block, 0, stream, x,
                                   y, ip);
            else if (deint)
                hipLaunchKernelGGL((view_interleave4_kernel<true, false>), grid, block, 0, stream,
                                   x, y, ip);
            else if (nt)
                hipLaunchKernelGGL((view_interleave4_kernel<false, true>), grid, block, 0, stream,
                                   x, y, ip);
            else
                hipLaunchKernelGGL((view_interleave4_kernel<false, false>), grid, block, 0, stream,
                                   x, y, ip);
            return check_launch("view_interleave4_kernel");
        }
    }

    // ---- tiled path: output-innermost dim is not the input-innermost one
    if (inner_coalesced_out && plain(inner) && inner.sr != 1 && total >= 4096) {
        // find the plain dim with the smallest positive input stride
        int in_inner = -1;
        for (int i = 0; i < c.rank; ++i)
            if (plain(c.d[i]) && c.d[i].sr > 0 &&
                (in_inner < 0 || c.d[i].sr < c.d[in_inner].sr))
                in_inner = i;
        if (in_inner >= 0 && in_inner != L && c.d[in_inner].sr < inner.sr) {
            int tsh[PET_HIP_MAX_RANK] = {0};
            // input run: ascending input stride until >= 64 elements
            std::vector<int> by_in, by_out;
            for (int i = 0; i < c.rank; ++i)
                if (plain(c.d[i]) && c.d[i].sr > 0)
                    by_in.push_back(i);
            std::sort(by_in.begin(), by_in.end(),
                      [&](int a, int b) { return c.d[a].sr < c.d[b].sr; });
            for (int i = 0; i < c.rank; ++i)
                if (plain(c.d[i]) && c.d[i].sr > 0 && c.d[i].os > 0)
                    by_out.push_back(i);
            std::sort(by_out.begin(), by_out.end(),
                      [&](int a, int b) { return c.d[a].os < c.d[b].os; });
            auto tile_dims = [&]() {
                int n = 0;
                for (int i = 0; i < c.rank; ++i)
                    n += tsh[i] > 0;
                return n;
            };
            auto tile_log = [&]() {
                int s = 0;
                for (int i = 0; i < c.rank; ++i)
                    s += tsh[i];
                return s;
            };
            auto run = [&](const std::vector<int> &order, int target_log) {
                int acc = 0;
                for (int d : order) {
                    if (acc >= target_log)
                        break;
                    int full = ceil_log2(c.d[d].ext);
                    int want = std::min(full, target_log - acc);
                    if (tsh[d] == 0 && tile_dims() >= kTileDims)
                        break;
                    tsh[d] = std::max(tsh[d], want);
                    acc += tsh[d];
                }
            };
            static const int tl_env =
                getenv("PET_HIP_VIEW_TILELOG") ? atoi(getenv("PET_HIP_VIEW_TILELOG")) : 0;
            // 8192-element tiles (512-byte runs on both sides) once there are thousands of them
            const int TL = tl_env ? tl_env : (total >= (1ll << 23) ? 13 : 12);
            const int RL = TL / 2;
            run(by_in, RL);
            run(by_out, RL);
            // grow towards 2^TL elements: alternate between the two orders
            bool grew = true;
            while (tile_log() < TL && grew) {
                grew = false;
                for (const std::vector<int> *ord : {&by_out, &by_in}) {
                    for (int d : *ord) {
                        if (tile_log() >= TL)
                            break;
                        if (tsh[d] < ceil_log2(c.d[d].ext) &&
                            (tsh[d] > 0 || tile_dims() < kTileDims)) {
                            tsh[d] += 1;
                            grew = true;
                            break;
                        }
                    }
                }
            }
            if (tile_log() <= TL && tile_dims() >= 2 && tile_dims() <= kTileDims) {
                TiledParams p;
                memset(&p, 0, sizeof(p));
                p.rank = c.rank;
                p.ibase = c.ibase;
                p.obase = c.obase;
                long long ngroups = 1;
                unsigned nt[PET_HIP_MAX_RANK], gstride[PET_HIP_MAX_RANK];
                for (int i = c.rank - 1; i >= 0; --i) {
                    const ViewDim &d = c.d[i];
                    nt[i] = (unsigned)((d.ext + (1 << tsh[i]) - 1) >> tsh[i]);
                    gstride[i] = (unsigned)ngroups;
                    ngroups *= nt[i];
                    if (ngroups >= (1ll << 31))
                        break;
                }
                for (int i = 0; i < c.rank && ngroups < (1ll << 31); ++i) {
                    const ViewDim &d = c.d[i];
                    p.is_tile[i] = tsh[i] > 0;
                    p.gdiv[i] = make_fastdiv(gstride[i]);
                    p.ntiles[i] = make_fastdiv(nt[i]);
                    p.has_div[i] = d.m < d.ext;
                    p.m[i] = make_fastdiv((unsigned)std::max(1, d.m));
                    p.lo[i] = d.lo;
                    p.hi[i] = d.hi;
                    p.os[i] = d.os;
                    p.sq[i] = d.sq;
                    p.sr[i] = d.sr;
                }
                std::vector<int> tin, tout;
                for (int d : by_in)
                    if (tsh[d] > 0)
                        tin.push_back(d);
                tout = tin;
                std::sort(tout.begin(), tout.end(),
                          [&](int a, int b) { return c.d[a].os < c.d[b].os; });
                p.ntd = (int)tin.size();
                int pos_of[PET_HIP_MAX_RANK] = {0};
                int pos = 0;
                for (int i = 0; i < p.ntd && ngroups < (1ll << 31); ++i) {
                    int d = tin[i];
                    p.in_gdiv[i] = make_fastdiv(gstride[d]);
                    p.in_nt[i] = make_fastdiv(nt[d]);
                    p.in_shift[i] = tsh[d];
                    p.in_ext[i] = c.d[d].ext;
                    p.in_sr[i] = c.d[d].sr;
                    pos_of[d] = pos;
                    pos += tsh[d];
                }
                for (int i = 0; i < p.ntd && ngroups < (1ll << 31); ++i) {
                    int d = tout[i];
                    p.out_gdiv[i] = make_fastdiv(gstride[d]);
                    p.out_nt[i] = make_fastdiv(nt[d]);
                    p.out_shift[i] = tsh[d];
                    p.out_ext[i] = c.d[d].ext;
                    p.out_os[i] = c.d[d].os;
                    p.out_to_in_pos[i] = pos_of[d];
                }
                p.tile_elems = 1 << pos;
                if (ngroups < (1ll << 31)) {
                    // can the global side move 16 bytes per lane?
                    auto vec_ok = [&](const std::vector<int> &ord, bool in_side) {
                        auto stride = [&](int d) { return in_side ? c.d[d].sr : c.d[d].os; };
                        const int d0 = ord[0];
                        size_t first_free = 1;
                        if (stride(d0) != 1)
                            return false;
                        if (tsh[d0] >= 2) {
                            if (c.d[d0].ext % 4)
                                return false;
                        } else {
                            // a 2-wide innermost dim: the next one must continue the run
                            if (c.d[d0].ext != 2 || ord.size() < 2 || stride(ord[1]) != 2 ||
                                c.d[ord[1]].ext % 2)
                                return false;
                            first_free = 2;
                        }
                        for (size_t i = first_free; i < ord.size(); ++i)
                            if (stride(ord[i]) % 4)
                                return false;
                        for (int i = 0; i < c.rank; ++i) {
                            if (tsh[i] > 0)
                                continue;
                            if (stride(i) % 4 || (in_side && c.d[i].m < c.d[i].ext && c.d[i].sq % 4))
                                return false;
                        }
                        const long long base = in_side ? c.ibase : c.obase;
                        const uintptr_t ptr = in_side ? (uintptr_t)x : (uintptr_t)y;
                        return base % 4 == 0 && ptr % 16 == 0;
                    };
                    const bool vin = vec_ok(tin, true), vout = vec_ok(tout, false);
                    const bool nt = stream_sized(total);
                    const dim3 grid((unsigned)ngroups);
                    const size_t lds_bytes =
                        (size_t)(p.tile_elems + p.tile_elems / 32 + 1) * sizeof(float);
#define PET_TILED(VI, VO, NTF) launch_tiled<VI, VO, NTF>(grid, lds_bytes, stream, x, y, p)
#define PET_TILED_NT(VI, VO)                                                                      \
    do {                                                                                          \
        if (nt)                                                                                   \
            PET_TILED(VI, VO, true);                                                              \
        else                                                                                      \
            PET_TILED(VI, VO, false);                                                             \
    } while (0)
                    if (vin && vout)
                        PET_TILED_NT(true, true);
                    else if (vin)
                        PET_TILED_NT(true, false);
                    else if (vout)
                        PET_TILED_NT(false, true);
                    else
                        PET_TILED_NT(false, false);
#undef PET_TILED_NT
#undef PET_TILED
                    return check_launch("view_tiled_kernel");
                }
            }
        }
    }

    // ---- direct path
    DirectParams p;
    memset(&p, 0, sizeof(p));
    p.rank = c.rank;
    p.ibase = c.ibase;
    p.obase = c.obase;
    bool vec = inner_coalesced_out && inner_coalesced_in && plain(inner) &&
               inner.ext % 4 == 0 && (c.ibase % 4 == 0) && (c.obase % 4 == 0) &&
               ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0);
    if (!plain(inner) && inner.os == 1 && inner.sr == 1 && inner.m >= inner.ext &&
        inner.ext % 4 == 0 && inner.lo % 4 == 0 && (inner.hi % 4 == 0 || inner.hi >= inner.ext) &&
        (c.ibase % 4 == 0) && (c.obase % 4 == 0) && ((uintptr_t)x % 16 == 0) &&
        ((uintptr_t)y % 16 == 0))
        vec = true; // windowed but 4-aligned innermost dim
    for (int i = 0; i < c.rank; ++i) {
        const ViewDim &d = c.d[i];
        if (i != L && (d.os % 4 || d.sr % 4 || (d.m < d.ext && d.sq % 4)))
            vec = false;
        p.has_div[i] = d.m < d.ext;
        p.m[i] = make_fastdiv((unsigned)std::max(1, d.m));
        p.lo[i] = d.lo;
        p.hi[i] = d.hi;
        p.os[i] = d.os;
        p.sq[i] = d.sq;
        p.sr[i] = d.sr;
        unsigned e = (unsigned)d.ext;
        if (i == L && vec)
            e /= 4;
        p.ext[i] = make_fastdiv(e);
    }
    if (vec) {
        p.lo[L] = c.d[L].lo;
        p.hi[L] = c.d[L].hi;
    }
    if (!vec && total % 4 == 0 && total >= 4096 && c.obase % 4 == 0 && (uintptr_t)y % 16 == 0) {
        // is the output dense (row-major over the iteration dims)?
        bool dense = true;
        long long expect = 1;
        for (int i = c.rank - 1; i >= 0; --i) {
            if (c.d[i].os != expect)
                dense = false;
            expect *= c.d[i].ext;
        }
        if (dense) {
            p.inner_contig = c.d[L].sr == 1 && c.d[L].m >= c.d[L].ext;
            p.total = (unsigned)(total / 4);
            const bool nt = stream_sized(total);
            if (p.inner_contig && c.d[L].ext >= 16 && (uintptr_t)x % 16 == 0) {
                RowStageParams rs;
                const long long words =
                    std::min<long long>((c.d[L].ext + 3) / 4 + 1, ROWSTAGE_TILE / 4 + 1);
                rs.cpr = make_fastdiv((unsigned)words);
                rs.zero = 0;
                for (int i = 0; i < c.rank; ++i)
                    if (c.d[i].lo > 0 || c.d[i].hi < std::min(c.d[i].ext, c.d[i].m))
                        rs.zero = 1;
                rs.total = (unsigned)total;
                const dim3 rgrid((unsigned)((total + ROWSTAGE_TILE - 1) / ROWSTAGE_TILE));
                if (nt)
                    hipLaunchKernelGGL(view_rowstage_kernel<true>, rgrid, dim3(256), 0, stream, x,
                                       y, p, rs);
                else
                    hipLaunchKernelGGL(view_rowstage_kernel<false>, rgrid, dim3(256), 0, stream,
                                       x, y, p, rs);
                return check_launch("view_rowstage_kernel");
            }
            const dim3 grid((unsigned)((p.total + 1023) / 1024)), block(256);
            if (nt)
                hipLaunchKernelGGL(view_gather4_kernel<true>, grid, block, 0, stream, x, y, p);
            else
                hipLaunchKernelGGL(view_gather4_kernel<false>, grid, block, 0, stream, x, y, p);
            return check_launch("view_gather4_kernel");
        }
    }
    long long items = vec ? total / 4 : total;
    p.total = (unsigned)items;
    // four items per thread once that still leaves every CU several workgroups
    const bool un4 = items >= 256ll * 4 * 2048;
    const bool nt = stream_sized(total);
    const unsigned per_wg = 256u * (un4 ? 4 : 1);
    const dim3 grid((unsigned)((items + per_wg - 1) / per_wg)), block(256);
#define PET_DIRECT(V, U, NTF)                                                                     \
    hipLaunchKernelGGL((view_direct_kernel<V, U, NTF>), grid, block, 0, stream, x, y, p)
    if (vec) {
        if (un4 && nt)
            PET_DIRECT(4, 4, true);
        else if (un4)
            PET_DIRECT(4, 4, false);
        else
            PET_DIRECT(4, 1, false);
    } else {
        if (un4 && nt)
            PET_DIRECT(1, 4, true);
        else if (un4)
            PET_DIRECT(1, 4, false);
        else
            PET_DIRECT(1, 1, false);
    }
#undef PET_DIRECT
    return check_launch("view_direct_kernel");
}

} // namespace pet
