// Parameters of the convolution kernels (conv.hip: LDS-staged tiles; direct.hip:
// register-fed tiles for small problems) and the raw-buffer helpers both use.
#pragma once
#include "mfma_common.h"

namespace pet {
namespace mfma {

// A 2-D operand read or written through strides (pet_hip_conv2d_view_f32): element
// (n, c, h, w) sits at batch(n) + c * sc + h * sh + w * sw floats from the base, where the
// batch index is taken apart into three factors, innermost first (extents ne0, ne1 and the
// rest), each with a stride of its own. A layout operator next to the convolution (space to
// batch in front, batch to space behind) becomes this addressing.
struct OperandView {
    int on;
    unsigned sc, sh, sw;
    unsigned ns[3];
    FastDiv fd_ne0, fd_ne1;
};

__device__ __forceinline__ unsigned view_batch_offset(const OperandView &v, unsigned n) {
    const unsigned q0 = fd_div(n, v.fd_ne0);
    const unsigned q1 = fd_div(q0, v.fd_ne1);
    return (n - q0 * v.fd_ne0.d) * v.ns[0] + (q0 - q1 * v.fd_ne1.d) * v.ns[1] + q1 * v.ns[2];
}

struct ConvParams {
    OperandView xv, yv; // plane and direct kernels, 2-D only; the residual is laid out like y
    const float *x, *w, *bias;
    const float *res; // optional residual, laid out like y: y = act(conv + bias + res)
    float *y;
    int N, C, T, H, W, F;
    int KT, R, S;
    int pt, ph, pw, st, sh, sw, dt, dh, dw;
    int G, cpg;
    int OT, OH, OW;
    int M;    // output channels per group
    int K;    // cpg * KT * R * S
    int NPIX; // N * OT * OH * OW
    int OPIX; // OT * OH * OW
    int act;
    int bias_mode; // 1: bias[f] per output channel, 2: bias[pixel] per output column
    int splitk;    // plane kernel: K steps are dealt to this many workgroups per tile
    int xcd_chunk; // plane kernel: tiles per XCD when the tile grid is dealt in bands (0: off)
    int xcd_mg;    // ... and how many M tiles wide a band is
    FastDiv fd_band, fd_mg, fd_splitk; // divisions by xcd_mg * grid.x, xcd_mg and splitk
    // stream-K (plane kernel): a 1-D grid of sk_wgs workgroups shares tiles * nit K steps
    // evenly; a workgroup runs its range as up to three segments of consecutive tiles
    int streamk, sk_units, sk_tiles_m;
    FastDiv fd_sk_wgs, fd_sk_nit, fd_sk_tm;
    int atomic_out; // partial sums are added into y with float atomics
    int vec_out;   // plane kernel: OPIX % 4 == 0 and y 16-byte aligned: 16-byte output words
    int wpacked;   // 3-D filters are stored kt-major, [kt][f][c/g][r][s] (plane kernel only)
    int sk_mode;   // split-K: 0 partial tiles + ordered sum in one launch, 1 atomics into y
    float *ws;     // split-K: partial tiles, [tile][split][register][thread]
    int *cnt;      // split-K: arrival counter per tile, zero between launches
    // caller-side fusion across launches (the *_ex entry points)
    int x_relu;     // the input is used as max(x, 0): its producer left ReLU to the readers
    int res_relu;   // the same for the residual operand
    int y_init;     // y already holds bias (or 0): a split launch does not initialise it
    int defer_relu; // a split launch leaves its ReLU to the readers of y
    int *dry_atomic; // not null: report whether the launch would accumulate into y, launch nothing
    int force_splitk;  // > 0: this many K shares per tile instead of the cost model's choice
    int force_streamk; // 0 / 1: stream-K off / on instead of the cost model's choice; -1: model
    int static_ws;   // split-K partial tiles and counters live in this file's static device
                     // array (the entry point that allocates nothing); implies the ordered sum
    int res_first;   // accumulating launch into an initialised y: the workgroup that holds a
                     // tile's first K step adds the residual along with its partial sums
    int w_shared;    // every group reads the filters of group 0 (a matmul whose A operand has
                     // one batch entry: an Extend of the lhs folded into the addressing)
    int bias_gstride; // bias_mode 2: floats between the groups' bias vectors (0: one for all)
    FastDiv fd_krs, fd_rs, fd_s;     // k -> (c, kt, r, s)
    FastDiv fd_opix, fd_ohw, fd_ow;  // pixel -> (n, ot, oh, ow)
};

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base) {
    // raw buffer, stride 0, 2 GiB of records, 32-bit float format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x80000000, 0x00020000);
}

constexpr unsigned kOob = 0x80000000u; // voffset that the range check rejects

// direct.hip: the register-fed kernel for contractions too small to fill the chip with
// LDS-staged tiles. Returns -1 when it does not apply (the caller goes on to the other
// kernels), else a pet_hip_status.
int try_launch_direct(const ConvParams &p, hipStream_t stream);

// stem.hip: 7x7 stride-2 filters over three channels, input patch and filter bank staged in
// LDS. Returns -1 when it does not apply, else a pet_hip_status.
int try_launch_stem(const ConvParams &p, hipStream_t stream);

// conv.hip: y = bias (+ residual) ahead of a launch that adds partial sums into y.
int launch_accumulate_init(const ConvParams &p, hipStream_t stream);

} // namespace mfma
} // namespace pet
