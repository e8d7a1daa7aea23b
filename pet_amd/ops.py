"""Operator calls on torch device tensors, each one a single C-ABI call.

torch only owns the memory and names the stream; shapes are worked out here
with the same rules as the reference's ``computeShape`` methods so callers can
allocate outputs. All tensors must be contiguous fp32 CUDA(HIP) tensors.
"""
import ctypes

import torch

from . import abi


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _chk(*ts):
    abi.init(torch.cuda.current_device())
    for t in ts:
        if t is None:
            continue
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
            raise ValueError("expected contiguous fp32 device tensors")


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def conv_out_dim(i, k, p, s, d):
    """ConvOp::computeShape, src/Graph/operator.cc:219-221."""
    return (i - (k - s) * d + 2 * p) // s if (i - (k - s) * d + 2 * p) >= 0 else -1


def interleave_view(q, c, hb, wb, d):
    """The strides under which a [q, c, d*hb, d*wb] tensor is the batch [(i, j, q), c, hb, wb]
    of its d*d pixel phases, entry (i*d + j)*q + image holding the pixels (d*y + i, d*x + j):
    PET's space-to-batch Transpose when the tensor is read, batch-to-space when written."""
    v = abi.ConvView()
    v.c_stride, v.h_stride, v.w_stride = d * hb * d * wb, d * d * wb, d
    v.n_extent[0], v.n_extent[1] = q, d
    v.n_stride[0], v.n_stride[1], v.n_stride[2] = c * d * hb * d * wb, 1, d * wb
    return v


def conv2d_view_supported(x_shape, w_shape, ph, pw, sh=1, sw=1, dh=1, dw=1):
    """Whether conv2d takes x_view / y_view for these (logical) shapes."""
    abi.init(torch.cuda.current_device())
    n, c, h, wd = x_shape
    f, cpg, r, s = w_shape
    yes = ctypes.c_int(0)
    abi.call("pet_hip_conv2d_view_supported", n, c, h, wd, f, r, s, ph, pw, sh, sw, dh, dw,
             c // cpg, ctypes.byref(yes))
    return bool(yes.value)


def conv2d(x, w, ph, pw, sh=1, sw=1, dh=1, dw=1, bias=None, act="none", out=None,
           residual=None, flags=0, x_view=None, x_shape=None, y_view=None):
    """act(conv(x, w) + bias + residual); residual has the output's shape. flags:
    pet_hip_call_flags (abi.Y_INITIALISED, DEFER_RELU, X_RELU, RES_RELU). x_view / y_view
    (abi.ConvView): x is read, y (and the residual) written through these strides, x_shape
    being the logical [n, c, h, w] of x and `out` a buffer of the output's size."""
    _chk(x, w, bias, out, residual)
    if x_view is not None or y_view is not None:
        n, c, h, wd = x_shape if x_view is not None else x.shape
        f, cpg, r, s = w.shape
        if cpg <= 0 or c % cpg:
            raise abi.PetHipError(1, "input channels not divisible by weight channels")
        oh, ow = conv_out_dim(h, r, ph, sh, dh), conv_out_dim(wd, s, pw, sw, dw)
        if x.numel() != n * c * h * wd:
            raise abi.PetHipError(1, "x does not hold the viewed shape")
        if out is None:
            if y_view is not None:
                raise abi.PetHipError(1, "a viewed output needs its buffer")
            out = torch.empty((n, f, max(oh, 0), max(ow, 0)), device=x.device,
                              dtype=torch.float32)
        if out.numel() != n * f * max(oh, 0) * max(ow, 0) or \
                (residual is not None and residual.numel() != out.numel()):
            raise abi.PetHipError(1, "output or residual of another size")
        abi.call("pet_hip_conv2d_view_f32", _ptr(x),
                 ctypes.byref(x_view) if x_view is not None else None, _ptr(w), _ptr(bias),
                 _ptr(residual), _ptr(out), ctypes.byref(y_view) if y_view is not None else None,
                 n, c, h, wd, f, r, s, ph, pw, sh, sw, dh, dw, c // cpg, abi.ACT[act], flags,
                 _stream())
        return out
    n, c, h, wd = x.shape
    f, cpg, r, s = w.shape
    if cpg <= 0 or c % cpg:
        raise abi.PetHipError(1, "input channels not divisible by weight channels")
    groups = c // cpg
    oh, ow = conv_out_dim(h, r, ph, sh, dh), conv_out_dim(wd, s, pw, sw, dw)
    if out is None:
        out = torch.empty((n, f, max(oh, 0), max(ow, 0)), device=x.device, dtype=torch.float32)
    if residual is not None and tuple(residual.shape) != tuple(out.shape):
        raise abi.PetHipError(1, "residual shape differs from the output's")
    if flags:
        abi.call("pet_hip_conv2d_ex_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out),
                 n, c, h, wd, f, r, s, ph, pw, sh, sw, dh, dw, groups, abi.ACT[act], flags,
                 _stream())
        return out
    if residual is not None:
        abi.call("pet_hip_conv2d_res_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(residual), _ptr(out),
                 n, c, h, wd, f, r, s, ph, pw, sh, sw, dh, dw, groups, abi.ACT[act], _stream())
        return out
    abi.call("pet_hip_conv2d_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), n, c, h, wd, f, r, s,
             ph, pw, sh, sw, dh, dw, groups, abi.ACT[act], _stream())
    return out


def conv2d_accumulates(x_shape, w_shape, ph, pw, sh=1, sw=1, dh=1, dw=1):
    """Whether conv2d on these shapes adds partial sums into its output with atomics."""
    abi.init(torch.cuda.current_device())
    n, c, h, wd = x_shape
    f, cpg, r, s = w_shape
    yes = ctypes.c_int(0)
    abi.call("pet_hip_conv2d_accumulates", n, c, h, wd, f, r, s, ph, pw, sh, sw, dh, dw, c // cpg,
             ctypes.byref(yes))
    return bool(yes.value)


def bmm_accumulates(b, m, n, k, transA=False, transB=False):
    abi.init(torch.cuda.current_device())
    yes = ctypes.c_int(0)
    abi.call("pet_hip_bmm_accumulates", int(transA), int(transB), b, m, n, k, ctypes.byref(yes))
    return bool(yes.value)


def bias_fill_batch(items):
    """items: (y, bias or None, outer, ch, inner) tuples; y[o][c][i] = bias[c], one launch."""
    arr = (abi.Fill * max(1, len(items)))()
    for i, (y, bias, outer, ch, inner) in enumerate(items):
        _chk(y, bias)
        arr[i] = abi.Fill(y.data_ptr(), 0 if bias is None else bias.data_ptr(), outer, ch, inner)
    abi.call("pet_hip_bias_fill_batch", arr, len(items), _stream())


class PackedFilters:
    """Constant 3-D filters in the kt-major layout of pet_hip_conv3d_pack_filters."""

    def __init__(self, data, shape):
        self.data, self.shape = data, tuple(shape)


def conv3d_pack_filters(w):
    """kt-major copy of constant filters [f, c/g, kt, r, s], or None when the shape
    has no such form (the caller keeps using the filters as they are). One-time
    weight preprocessing, outside any timed or captured region."""
    _chk(w)
    f, cpg, kt, r, s = w.shape
    packed = torch.empty_like(w)
    rc = abi.status("pet_hip_conv3d_pack_filters", _ptr(w), _ptr(packed), f, cpg, kt, r, s,
                    _stream())
    if rc == 2:     # PET_HIP_ERR_UNSUPPORTED
        return None
    if rc != 0:
        raise abi.PetHipError(rc, abi.last_error())
    return PackedFilters(packed, w.shape)


def conv3d(x, w, pad, stride=(1, 1, 1), dil=(1, 1, 1), bias=None, act="none", out=None,
           residual=None):
    """w: filters [f, c/g, kt, r, s], or a PackedFilters made from them."""
    entry = "pet_hip_conv3d_f32"
    if isinstance(w, PackedFilters):
        entry, wshape, w = "pet_hip_conv3d_packed_f32", w.shape, w.data
    else:
        wshape = w.shape
    _chk(x, w, bias, out, residual)
    n, c, t, h, wd = x.shape
    f, cpg, kt, r, s = wshape
    if cpg <= 0 or c % cpg:
        raise abi.PetHipError(1, "input channels not divisible by weight channels")
    groups = c // cpg
    ot = conv_out_dim(t, kt, pad[0], stride[0], dil[0])
    oh = conv_out_dim(h, r, pad[1], stride[1], dil[1])
    ow = conv_out_dim(wd, s, pad[2], stride[2], dil[2])
    if out is None:
        out = torch.empty((n, f, ot, oh, ow), device=x.device, dtype=torch.float32)
    if residual is not None:
        if tuple(residual.shape) != tuple(out.shape):
            raise abi.PetHipError(1, "residual shape differs from the output's")
        abi.call("pet_hip_conv3d_res_f32", _ptr(x), _ptr(w),
                 int(entry == "pet_hip_conv3d_packed_f32"), _ptr(bias), _ptr(residual), _ptr(out),
                 n, c, t, h, wd, f, kt, r, s, *pad, *stride, *dil, groups, abi.ACT[act], _stream())
        return out
    abi.call(entry, _ptr(x), _ptr(w), _ptr(bias), _ptr(out), n, c, t, h, wd, f, kt,
             r, s, *pad, *stride, *dil, groups, abi.ACT[act], _stream())
    return out


def matmul(A, B, transA=False, transB=False, bias=None, act="none", out=None, residual=None,
           flags=0):
    """MatmulOp on [b, ., .] tensors (MatmulOp::computeShape, operator.cc:717-726);
    with residual: act(A @ B + bias + residual). flags: pet_hip_call_flags (abi.A_SHARED:
    A is [1, ., .] and multiplies every batch entry of B; abi.BIAS_PER_BATCH: bias [b, n])."""
    _chk(A, B, bias, out, residual)
    b = B.shape[0] if flags & abi.A_SHARED else A.shape[0]
    if flags & abi.A_SHARED and A.shape[0] != 1:
        raise abi.PetHipError(1, "a shared lhs has one batch entry")
    if flags & abi.BIAS_PER_BATCH and (bias is None or bias.numel() != b * (
            B.shape[1] if transB else B.shape[2])):
        raise abi.PetHipError(1, "a per-batch bias holds b * n values")
    m = A.shape[2] if transA else A.shape[1]
    k = A.shape[1] if transA else A.shape[2]
    n = B.shape[1] if transB else B.shape[2]
    kb = B.shape[2] if transB else B.shape[1]
    if B.shape[0] != b or kb != k:
        raise abi.PetHipError(1, "matmul shapes do not agree")
    if out is None:
        out = torch.empty((b, m, n), device=A.device, dtype=torch.float32)
    if residual is not None and residual.numel() != out.numel():
        raise abi.PetHipError(1, "residual size differs from the output's")
    if flags:
        abi.call("pet_hip_bmm_ex_f32", int(transA), int(transB), b, m, n, k, _ptr(A), _ptr(B),
                 _ptr(out), _ptr(bias), _ptr(residual), abi.ACT[act], flags, _stream())
        return out
    if residual is not None:
        abi.call("pet_hip_bmm_res_f32", int(transA), int(transB), b, m, n, k, _ptr(A), _ptr(B),
                 _ptr(out), _ptr(bias), _ptr(residual), abi.ACT[act], _stream())
        return out
    abi.call("pet_hip_bmm_f32", int(transA), int(transB), b, m, n, k, _ptr(A), _ptr(B), _ptr(out),
             _ptr(bias), abi.ACT[act], _stream())
    return out


def conv_trans_out_dim(i, k, p, s, d, op):
    """ConvTransOp::computeShape, src/Graph/operator.cc:1066-1067."""
    return (i - 1) * s - 2 * p + d * (k - 1) + op + 1


def conv_trans(x, w, ph, pw, sh=1, sw=1, dh=1, dw=1, oph=0, opw=0, bias=None, act="none",
               out=None):
    """ConvTransOp: x NHWF [n,h,w,f], w RSFC [r,s,f,c] -> NHWC [n,oh,ow,c]."""
    _chk(x, w, bias, out)
    n, h, wd, f = x.shape
    r, s, f2, c = w.shape
    if f != f2:
        raise abi.PetHipError(1, "input features differ from the weight's")
    oh = conv_trans_out_dim(h, r, ph, sh, dh, oph)
    ow = conv_trans_out_dim(wd, s, pw, sw, dw, opw)
    if out is None:
        out = torch.empty((n, max(oh, 0), max(ow, 0), c), device=x.device, dtype=torch.float32)
    abi.call("pet_hip_conv_trans_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), n, h, wd, f, r, s,
             c, ph, pw, sh, sw, dh, dw, oph, opw, abi.ACT[act], _stream())
    return out


def g2bmm(A, B, width, dilation=1, out=None):
    """G2BMMOp: A, B [bs,m,k] -> [bs,m,2*width+1]."""
    _chk(A, B, out)
    bs, m, k = A.shape
    if tuple(B.shape) != tuple(A.shape):
        raise abi.PetHipError(1, "g2bmm operands differ in shape")
    if out is None:
        out = torch.empty((bs, m, 2 * width + 1), device=A.device, dtype=torch.float32)
    abi.call("pet_hip_g2bmm_f32", _ptr(A), _ptr(B), _ptr(out), bs, m, k, width, dilation,
             _stream())
    return out


def gbmml(A, B, dilation=1, out=None):
    """GBMMLOp: A [bs,m,2w+1], B [bs,m,n] -> [bs,m,n]."""
    _chk(A, B, out)
    bs, m, band = A.shape
    if band % 2 == 0 or tuple(B.shape[:2]) != (bs, m):
        raise abi.PetHipError(1, "gbmml operands do not agree")
    n = B.shape[2]
    if out is None:
        out = torch.empty((bs, m, n), device=A.device, dtype=torch.float32)
    abi.call("pet_hip_gbmml_f32", _ptr(A), _ptr(B), _ptr(out), bs, m, (band - 1) // 2, n,
             dilation, _stream())
    return out


def attention(q, k, v, heads, scale=1.0, scale_dev=None, out=None):
    """softmax(scale * Q_h K_h^T) V_h for every head, on [seq, heads*dh] (or [batch, seq,
    heads*dh]) matrices; q, k, v may be row-strided views (slabs of a merged projection)."""
    abi.init(torch.cuda.current_device())
    for t in (q, k, v):
        if not (t.is_cuda and t.dtype == torch.float32 and t.stride(-1) == 1):
            raise ValueError("expected fp32 device matrices with contiguous rows")
    q3, k3, v3 = (t if t.dim() == 3 else t.unsqueeze(0) for t in (q, k, v))
    batch, seq, width = q3.shape
    if width % heads or tuple(k3.shape) != tuple(q3.shape) or tuple(v3.shape) != tuple(q3.shape):
        raise abi.PetHipError(1, "attention operands do not agree")
    if out is None:
        out = torch.empty(tuple(q.shape), device=q.device, dtype=torch.float32)
    o3 = out if out.dim() == 3 else out.unsqueeze(0)
    abi.call("pet_hip_attention_f32", _ptr(q3), _ptr(k3), _ptr(v3), _ptr(o3), batch, heads, seq,
             width // heads, q3.stride(1), k3.stride(1), v3.stride(1), o3.stride(1),
             q3.stride(0), k3.stride(0), v3.stride(0), o3.stride(0), float(scale),
             _ptr(scale_dev), _stream())
    return out


class ExprProgram:
    """An index-expression program (see pet_hip.h) with its device copy."""

    def __init__(self, code):
        abi.init(torch.cuda.current_device())
        self.code = abi.ints(code)
        self.ncode = len(code)
        dev = ctypes.c_void_p(0)
        abi.call("pet_hip_expr_program_create", self.code, self.ncode, ctypes.byref(dev))
        self.dev = dev
        at = 2
        for _ in range(code[1]):
            at += 1 + code[at]
        self.out_shape = tuple(code[at + 1:at + 1 + code[at]])

    def __del__(self):
        # at interpreter exit the module globals may already be gone
        if getattr(self, "dev", None) is not None and self.dev.value and abi is not None:
            abi.status("pet_hip_free", self.dev)


def expr(program, inputs, out=None):
    """MemBoundOp: out[pos] = program(pos) over the output shape in the program's header."""
    _chk(out, *inputs)
    if out is None:
        out = torch.empty(program.out_shape, device=inputs[0].device, dtype=torch.float32)
    ptrs = (ctypes.c_void_p * max(1, len(inputs)))(*[t.data_ptr() for t in inputs])
    abi.call("pet_hip_expr_f32", program.code, program.ncode, program.dev, ptrs, len(inputs),
             _ptr(out), _stream())
    return out


def transpose_params(in_dims, split, after, factor):
    """TransposeOp::setParam (include/operator.h:1124-1144) and the flat-dim
    rule of TransposeOp::computeShape (src/Graph/operator.cc:2340-2381).
    Returns (flat_dims, perm, out_dims) or None when the split does not divide."""
    items = [list(a) if isinstance(a, (list, tuple)) else [a] for a in after]
    if split >= 0:
        if factor == 0:
            return None
        items = [[(split + 1) if i == -1 else (i + 1 if i > split else i) for i in it]
                 for it in items]
    flat = []
    for i, d in enumerate(in_dims):
        if i != split:
            flat.append(d)
        elif factor > 0:
            if d % factor or d < factor:
                return None
            flat += [d // factor, factor]
        else:
            if d % (-factor) or d < -factor:
                return None
            flat += [-factor, d // (-factor)]
    perm = [i for it in items for i in it]
    if sorted(perm) != list(range(len(flat))) or sum(len(it) > 1 for it in items) > 1:
        return None
    out = []
    for it in items:
        e = 1
        for i in it:
            e *= flat[i]
        out.append(e)
    return flat, perm, out


def transpose(x, split, after, factor=2, out=None):
    """TransposeOp(input, split, after, factor)."""
    _chk(x, out)
    prm = transpose_params(list(x.shape), split, after, factor)
    if prm is None:
        return None
    flat, perm, oshape = prm
    if out is None:
        out = torch.empty(oshape, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_transpose", _ptr(x), _ptr(out), abi.ints(flat), abi.ints(perm), len(flat),
             _stream())
    return out


def permute_flat(x, flat, perm, out=None):
    _chk(x, out)
    if out is None:
        out = torch.empty([flat[i] for i in perm], device=x.device, dtype=torch.float32)
    abi.call("pet_hip_transpose", _ptr(x), _ptr(out), abi.ints(flat), abi.ints(perm), len(flat),
             _stream())
    return out


def _encode_chain(micro_ops):
    enc, perms = [], []
    for op in micro_ops:
        if op[0] == "split":
            enc += [0, op[1], op[2], op[3], op[4], 0]
        elif op[0] == "reorder":
            enc += [1, 0, 0, 0, 0, 0]
            perms += list(op[1])
        elif op[0] == "fuse":
            enc += [2, op[1], op[2], op[3], 0, 0]
        else:
            raise ValueError(op[0])
    return enc, perms


def trans_chain(x, micro_ops, out=None):
    """A TransSplit / TransReorder / TransFuse chain (src/Transpose/transpose.cc)."""
    _chk(x, out)
    enc, perms = _encode_chain(micro_ops)
    odims = (ctypes.c_int * 8)()
    ork = ctypes.c_int(0)
    args = (abi.ints(x.shape), x.dim(), abi.ints(enc), len(micro_ops), abi.ints(perms), odims,
            ctypes.byref(ork), _stream())
    abi.call("pet_hip_trans_chain", _ptr(x), ctypes.c_void_p(0), *args)
    oshape = [odims[i] for i in range(ork.value)]
    if out is None:
        out = torch.empty(oshape, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_trans_chain", _ptr(x), _ptr(out), *args)
    return out


def split_sizes(dim_size, sizes=None, num=None):
    """SplitOp::computeShapeV ratio rule, src/Graph/operator.cc:2074-2101."""
    if not sizes:
        if num is None or num <= 0:
            return None
        sizes = [1] * num
    total = sum(sizes)
    if total <= 0 or dim_size % total:
        return None
    return [dim_size // total * s for s in sizes]


def split(x, dim, sizes=None, num=None):
    _chk(x)
    szs = split_sizes(x.shape[dim], sizes, num)
    if szs is None:
        return None
    outs = []
    for s in szs:
        shp = list(x.shape)
        shp[dim] = s
        outs.append(torch.empty(shp, device=x.device, dtype=torch.float32))
    ptrs = (ctypes.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
    abi.call("pet_hip_split", _ptr(x), ptrs, len(outs), abi.ints(x.shape), x.dim(), dim,
             abi.ints(szs), _stream())
    return outs


def concat(xs, dim, out=None):
    _chk(*xs)
    shp = list(xs[0].shape)
    shp[dim] = sum(x.shape[dim] for x in xs)
    if out is None:
        out = torch.empty(shp, device=xs[0].device, dtype=torch.float32)
    ptrs = (ctypes.c_void_p * len(xs))(*[x.data_ptr() for x in xs])
    abi.call("pet_hip_concat", ptrs, len(xs), _ptr(out), abi.ints(shp), len(shp), dim,
             abi.ints([x.shape[dim] for x in xs]), _stream())
    return out


def pad(x, begin, end, out=None):
    _chk(x, out)
    shp = [d + b + e for d, b, e in zip(x.shape, begin, end)]
    if out is None:
        out = torch.empty(shp, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_pad", _ptr(x), _ptr(out), abi.ints(x.shape), abi.ints(begin), abi.ints(end),
             x.dim(), _stream())
    return out


def slice_(x, begin, end, out=None):
    _chk(x, out)
    shp = [max(d - b - e, 0) for d, b, e in zip(x.shape, begin, end)]
    if out is None:
        out = torch.empty(shp, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_slice", _ptr(x), _ptr(out), abi.ints(x.shape), abi.ints(begin),
             abi.ints(end), x.dim(), _stream())
    return out


def extend(x, dim, num, out=None):
    _chk(x, out)
    shp = list(x.shape)
    shp[dim] *= num + 1
    if out is None:
        out = torch.empty(shp, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_extend", _ptr(x), _ptr(out), abi.ints(x.shape), x.dim(), dim, num, _stream())
    return out


def eltwise(op, xs, out_shape=None, out=None):
    _chk(*xs)
    if out is None:
        out = torch.empty(out_shape, device=xs[0].device, dtype=torch.float32)
    ptrs = (ctypes.c_void_p * len(xs))(*[x.data_ptr() for x in xs])
    sizes = (ctypes.c_size_t * len(xs))(*[x.numel() for x in xs])
    abi.call("pet_hip_eltwise", abi.ELT[op], ptrs, sizes, len(xs), _ptr(out), out.numel(),
             _stream())
    return out


def activation(x, act, out=None):
    _chk(x, out)
    if out is None:
        out = torch.empty_like(x)
    abi.call("pet_hip_activation", _ptr(x), _ptr(out), x.numel(), abi.ACT[act], _stream())
    return out


def pow_(x, power, out=None):
    """PowOp (operator.cc:3330-3343): `power` copies of x multiplied up from 1."""
    _chk(x, out)
    if out is None:
        out = torch.empty_like(x)
    abi.call("pet_hip_pow", _ptr(x), _ptr(out), x.numel(), int(power), _stream())
    return out


def batchnorm(x, scale, bias, mean, var, eps=1e-5, out=None):
    """BatchNormOp (operator.cc:2660-2681): inference statistics, channel axis 1."""
    _chk(x, scale, bias, mean, var, out)
    ch = x.shape[1]
    if any(t.numel() != ch for t in (scale, bias, mean, var)):
        raise abi.PetHipError(1, "per-channel vectors must have %d elements" % ch)
    inner = 1
    for d in x.shape[2:]:
        inner *= d
    if out is None:
        out = torch.empty_like(x)
    abi.call("pet_hip_batchnorm", _ptr(x), _ptr(scale), _ptr(bias), _ptr(mean), _ptr(var),
             _ptr(out), x.shape[0], ch, inner, float(eps), _stream())
    return out


def gather(x, indices, axis, out=None):
    """GatherOp (shape rule operator.cc:3420-3428): the index dims lead the output.
    indices: int32 or float32 (holding integers) tensor on the device."""
    if indices.dtype not in (torch.int32, torch.float32):
        raise abi.PetHipError(1, "indices must be int32 or float32")
    _chk(x, out)
    if not (indices.is_cuda and indices.is_contiguous()):
        raise abi.PetHipError(1, "indices must be a contiguous device tensor")
    pre = 1
    for d in x.shape[:axis]:
        pre *= d
    post = 1
    for d in x.shape[axis + 1:]:
        post *= d
    shp = list(indices.shape) + list(x.shape[:axis]) + list(x.shape[axis + 1:])
    if out is None:
        out = torch.empty(shp, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_gather", _ptr(x), indices.data_ptr(), int(indices.dtype == torch.float32),
             _ptr(out), pre, x.shape[axis], post, indices.numel(), _stream())
    return out


def reduce_mean(x, axis, out=None):
    """ReduceMeanOp (shape rule operator.cc:3454-3458): mean over one axis, kept as 1."""
    _chk(x, out)
    outer = 1
    for d in x.shape[:axis]:
        outer *= d
    inner = 1
    for d in x.shape[axis + 1:]:
        inner *= d
    shp = list(x.shape)
    shp[axis] = 1
    if out is None:
        out = torch.empty(shp, device=x.device, dtype=torch.float32)
    abi.call("pet_hip_reduce_mean", _ptr(x), _ptr(out), outer, x.shape[axis], inner, _stream())
    return out


def bias_act(x, bias, act="none", ch_axis=1, out=None):
    _chk(x, bias, out)
    outer = 1
    for d in x.shape[:ch_axis]:
        outer *= d
    inner = 1
    for d in x.shape[ch_axis + 1:]:
        inner *= d
    if out is None:
        out = torch.empty_like(x)
    abi.call("pet_hip_bias_act", _ptr(x), _ptr(bias), _ptr(out), outer, x.shape[ch_axis], inner,
             abi.ACT[act], _stream())
    return out


def pool2d(x, kh, kw, ph, pw, sh, sw, dh=1, dw=1, mode="max", out=None, flags=0):
    """flags: abi.X_RELU pools max(x, 0)."""
    _chk(x, out)
    n, c, h, w = x.shape
    oh = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    if out is None:
        out = torch.empty((n, c, oh, ow), device=x.device, dtype=torch.float32)
    abi.call("pet_hip_pool2d_ex", _ptr(x), _ptr(out), n, c, h, w, kh, kw, ph, pw, sh, sw, dh, dw,
             0 if mode == "max" else 1, flags, _stream())
    return out


def softmax(x, out=None):
    _chk(x, out)
    if out is None:
        out = torch.empty_like(x)
    cols = x.shape[-1]
    abi.call("pet_hip_softmax", _ptr(x), _ptr(out), x.numel() // cols, cols, _stream())
    return out


def layernorm(x, gamma, beta, eps=1e-5, out=None):
    _chk(x, gamma, beta, out)
    if out is None:
        out = torch.empty_like(x)
    cols = x.shape[-1]
    abi.call("pet_hip_layernorm", _ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), x.numel() // cols,
             cols, ctypes.c_float(eps), _stream())
    return out
