// The "view copy" engine every layout operator lowers into.
//
// A ViewDesc names an iteration space of up to 8 dims. For an index vector idx
// the engine writes
//     out[obase + sum_d idx[d] * os[d]] =
//         valid ? in[ibase + sum_d (q_d * sq[d] + r_d * sr[d])] : 0
// with q_d = idx[d] / m[d], r_d = idx[d] % m[d] and valid = all_d(lo[d] <= r_d < hi[d]).
// Transposes, halo splits, drop/pad fuses, split, concat, pad, slice and extend
// are all instances (strides, one div/mod level per dim, a validity window).
#pragma once
#include <cstdint>

#include "common.h"

namespace pet {

struct ViewDim {
    int ext; // extent of the iteration dim
    int m;   // divisor of the one div/mod level (>= ext means none)
    int lo, hi; // validity window on r
    long long os; // output stride
    long long sq; // input stride of q
    long long sr; // input stride of r
};

struct ViewDesc {
    int rank;
    ViewDim d[PET_HIP_MAX_RANK];
    long long ibase, obase;
};

// Launches the best kernel for the view (after canonicalisation). `in_elems` /
// `out_elems` are the sizes of the two buffers, used for a host-side bounds
// check of the whole index space before anything is launched.
int launch_view_copy(const float *x, float *y, ViewDesc v, long long in_elems,
                     long long out_elems, hipStream_t stream);

// Row-major strides helper.
inline void row_major_strides(const int *dims, int rank, long long *strides) {
    long long s = 1;
    for (int i = rank - 1; i >= 0; --i) {
        strides[i] = s;
        s *= dims[i];
    }
}

} // namespace pet
