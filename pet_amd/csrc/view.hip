// View-copy engine: canonicalisation, kernel selection and the two kernels
// (direct and LDS-tiled) behind every layout operator.
#include "view.h"

#include <algorithm>
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
};

// One work item = VEC consecutive elements of the innermost iteration dim.
// With VEC == 4 the host has checked that the four elements are contiguous and
// 16-byte aligned on both sides and share one validity result.
template <int VEC>
__global__ __launch_bounds__(256) void view_direct_kernel(const float *__restrict__ x,
                                                          float *__restrict__ y,
                                                          DirectParams p) {
    unsigned t = blockIdx.x * 256u + threadIdx.x;
    const unsigned step = gridDim.x * 256u;
    for (; t < p.total; t += step) {
        unsigned rem = t;
        long long io = p.ibase, oo = p.obase;
        bool ok = true;
#pragma unroll
        for (int d = PET_HIP_MAX_RANK - 1; d >= 0; --d) {
            if (d < p.rank) {
                unsigned q = fd_div(rem, p.ext[d]);
                unsigned idx = rem - q * p.ext[d].d;
                rem = q;
                if (d == p.rank - 1)
                    idx *= VEC;
                oo += (long long)idx * p.os[d];
                unsigned r = idx;
                if (p.has_div[d]) {
                    unsigned qq = fd_div(idx, p.m[d]);
                    r = idx - qq * p.m[d].d;
                    io += (long long)qq * p.sq[d];
                }
                io += (long long)r * p.sr[d];
                ok = ok && ((int)r >= p.lo[d]) && ((int)r < p.hi[d]);
            }
        }
        if (VEC == 4) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (ok)
                v = *reinterpret_cast<const float4 *>(x + io);
            *reinterpret_cast<float4 *>(y + oo) = v;
        } else {
            y[oo] = ok ? x[io] : 0.f;
        }
    }
}

// ---- LDS-tiled kernel --------------------------------------------------------
// Up to 4 tile dims with power-of-two tile extents. Elements are read in
// "input order" (tile dims sorted by input stride, so consecutive lanes read
// consecutive addresses), parked in LDS, and written in "output order" (sorted
// by output stride). Dims outside the tile are handled by the grid.
constexpr int kTileMax = 4096;
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

__global__ __launch_bounds__(256) void view_tiled_kernel(const float *__restrict__ x,
                                                         float *__restrict__ y,
                                                         TiledParams p) {
    __shared__ float lds[kTileMax + kTileMax / 32];
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
    // load phase: consecutive lanes walk the tile in input order
    for (int t = threadIdx.x; t < p.tile_elems; t += 256) {
        int remt = t;
        long long io = ibase;
        bool ok = wg_ok;
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
        float v = 0.f;
        if (ok)
            v = x[io];
        lds[t + (t >> 5)] = v;
    }
    __syncthreads();
    // store phase: consecutive lanes walk the tile in output order
    for (int t = threadIdx.x; t < p.tile_elems; t += 256) {
        int remt = t;
        long long oo = obase;
        int lin = 0;
        bool ok = true;
#pragma unroll
        for (int i = 0; i < kTileDims; ++i) {
            if (i < p.ntd) {
                int c = remt & ((1 << p.out_shift[i]) - 1);
                remt >>= p.out_shift[i];
                int idx = org_out[i] + c;
                ok = ok && idx < p.out_ext[i];
                oo += (long long)idx * p.out_os[i];
                lin += c << p.out_to_in_pos[i];
            }
        }
        if (ok)
            y[oo] = lds[lin + (lin >> 5)];
    }
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
    if (!x || !y)
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
            run(by_in, 6);
            run(by_out, 6);
            // grow towards 4096 elements: alternate between the two orders
            bool grew = true;
            while (tile_log() < 12 && grew) {
                grew = false;
                for (const std::vector<int> *ord : {&by_out, &by_in}) {
                    for (int d : *ord) {
                        if (tile_log() >= 12)
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
            if (tile_log() <= 12 && tile_dims() >= 2 && tile_dims() <= kTileDims) {
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
                    hipLaunchKernelGGL(view_tiled_kernel, dim3((unsigned)ngroups), dim3(256), 0,
                                       stream, x, y, p);
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
    long long items = vec ? total / 4 : total;
    p.total = (unsigned)items;
    unsigned grid = (unsigned)std::min<long long>((items + 255) / 256, 1 << 20);
    if (vec)
        hipLaunchKernelGGL(view_direct_kernel<4>, dim3(grid), dim3(256), 0, stream, x, y, p);
    else
        hipLaunchKernelGGL(view_direct_kernel<1>, dim3(grid), dim3(256), 0, stream, x, y, p);
    return check_launch("view_direct_kernel");
}

} // namespace pet
