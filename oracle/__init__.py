"""TEST INFRASTRUCTURE ONLY -- numpy front-end of the CPU oracle.

Loads ``libpet_oracle.so`` (built from ``pet_oracle.c`` by ``make -C oracle``) and
wraps each C function with shape handling. The shipped package never imports this
module; only ``tests/``, ``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of
``bench.py`` do, and only as the checker.

Every wrapper takes ``uint32`` or ``float32`` arrays and picks the matching tier
(``*_u32`` wraps like the reference's VType, ``*_f32`` accumulates in fp64).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpet_oracle.so")
_lib = None

_c_int_p = ctypes.POINTER(ctypes.c_int)


def build():
    """Compile the oracle with the committed Makefile."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_conv_out_dim.restype = ctypes.c_int
        _lib.oracle_num_threads.restype = ctypes.c_int
        for suf in ("u32", "f32"):
            getattr(_lib, "oracle_conv2d_point_" + suf).restype = (
                ctypes.c_uint32 if suf == "u32" else ctypes.c_float)
    return _lib


def num_threads():
    return lib().oracle_num_threads()


def _tier(*arrays):
    dt = arrays[0].dtype
    for a in arrays:
        if a.dtype != dt:
            raise TypeError("mixed dtypes")
    if dt == np.uint32:
        return "u32"
    if dt == np.float32:
        return "f32"
    raise TypeError("oracle works on uint32 or float32, got %s" % dt)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _ints(v):
    arr = (ctypes.c_int * max(1, len(v)))(*[int(i) for i in v])
    return arr


def _c(a):
    return np.ascontiguousarray(a)


# ---------------------------------------------------------------- shape rules

def conv_out_dim(i, k, p, s, d):
    """ConvOp::computeShape, src/Graph/operator.cc:219-221."""
    return lib().oracle_conv_out_dim(int(i), int(k), int(p), int(s), int(d))


def transpose_params(in_dims, split, after, factor):
    """TransposeOp::setParam + flat-dim rule.

    include/operator.h:1124-1144 renumbers ``after``: with a split, entries
    greater than ``split`` move up by one and ``-1`` becomes ``split + 1``;
    src/Graph/operator.cc:2177-2194 turns the split dim into ``(d/f, f)`` when
    ``factor > 0`` and ``(-f, d/-f)`` when ``factor < 0``.

    ``after`` is a list whose items are ints or lists of ints (a merge).
    Returns (flat_dims, after_flat, out_dims) or None when not divisible
    (operator.cc:2184-2191 returns nullptr, :2348-2351 marks Invalid).
    """
    items = [list(a) if isinstance(a, (list, tuple)) else [a] for a in after]
    if split >= 0:
        if factor == 0:
            return None
        items = [[(split + 1) if i == -1 else (i + 1 if i > split else i)
                  for i in it] for it in items]
    flat = []
    for i, d in enumerate(in_dims):
        if i == split:
            if factor > 0:
                if d % factor or d < factor:
                    return None
                flat += [d // factor, factor]
            else:
                if d % (-factor) or d < -factor:
                    return None
                flat += [-factor, d // (-factor)]
        else:
            flat.append(d)
    after_flat = [i for it in items for i in it]
    if sorted(after_flat) != list(range(len(flat))):
        return None
    if sum(1 for it in items if len(it) > 1) > 1:
        return None
    out = [int(np.prod([flat[i] for i in it])) for it in items]
    return flat, after_flat, out


def split_sizes(dim_size, sizes=None, num=None):
    """SplitOp::computeShapeV, src/Graph/operator.cc:2074-2101: ``sizes`` are
    ratios -- out_i = dim / sum(sizes) * sizes_i; equal split when only ``num``
    is given. Returns None when not divisible."""
    if not sizes:
        if num is None or num <= 0:
            return None
        sizes = [1] * num
    total = sum(sizes)
    if total <= 0 or dim_size % total:
        return None
    return [dim_size // total * s for s in sizes]


# ------------------------------------------------------------------ operators

def conv2d(x, w, ph, pw, sh=1, sw=1, dh=1, dw=1):
    x, w = _c(x), _c(w)
    t = _tier(x, w)
    n, c, h, wd = x.shape
    f, cpg, r, s = w.shape
    oh = conv_out_dim(h, r, ph, sh, dh)
    ow = conv_out_dim(wd, s, pw, sw, dw)
    y = np.empty((n, f, oh, ow), dtype=x.dtype)
    rc = getattr(lib(), "oracle_conv2d_" + t)(
        _p(x), _p(w), _p(y), n, c, h, wd, f, cpg, r, s, ph, pw, sh, sw, dh, dw,
        oh, ow)
    return None if rc else y


def conv2d_point(x, w, ph, pw, sh, sw, dh, dw, pos):
    x, w = _c(x), _c(w)
    t = _tier(x, w)
    n, c, h, wd = x.shape
    f, cpg, r, s = w.shape
    return getattr(lib(), "oracle_conv2d_point_" + t)(
        _p(x), _p(w), n, c, h, wd, f, cpg, r, s, ph, pw, sh, sw, dh, dw,
        *[int(v) for v in pos])


def conv3d(x, w, pad, stride=(1, 1, 1), dil=(1, 1, 1)):
    x, w = _c(x), _c(w)
    t = _tier(x, w)
    n, c, tt, h, wd = x.shape
    f, cpg, kt, r, s = w.shape
    ot = conv_out_dim(tt, kt, pad[0], stride[0], dil[0])
    oh = conv_out_dim(h, r, pad[1], stride[1], dil[1])
    ow = conv_out_dim(wd, s, pad[2], stride[2], dil[2])
    y = np.empty((n, f, ot, oh, ow), dtype=x.dtype)
    rc = getattr(lib(), "oracle_conv3d_" + t)(
        _p(x), _p(w), _p(y), n, c, tt, h, wd, f, cpg, kt, r, s, *pad, *stride,
        *dil, ot, oh, ow)
    return None if rc else y


def matmul(A, B, transA=False, transB=False):
    A, B = _c(A), _c(B)
    t = _tier(A, B)
    b = A.shape[0]
    m = A.shape[2] if transA else A.shape[1]
    k = A.shape[1] if transA else A.shape[2]
    n = B.shape[1] if transB else B.shape[2]
    C = np.empty((b, m, n), dtype=A.dtype)
    getattr(lib(), "oracle_matmul_" + t)(_p(A), _p(B), _p(C), b, m, n, k,
                                         int(transA), int(transB))
    return C


def conv_trans_out_dim(i, k, p, s, d, op):
    """ConvTransOp::computeShape, src/Graph/operator.cc:1066-1067."""
    return (i - 1) * s - 2 * p + d * (k - 1) + op + 1


def conv_trans(x, w, ph, pw, sh=1, sw=1, dh=1, dw=1, oph=0, opw=0):
    """ConvTransOp::compute: x NHWF [n,h,w,f], w RSFC [r,s,f,c] -> NHWC [n,oh,ow,c]."""
    x, w = _c(x), _c(w)
    t = _tier(x, w)
    n, h, wd, f = x.shape
    r, s, f2, c = w.shape
    assert f == f2
    oh = conv_trans_out_dim(h, r, ph, sh, dh, oph)
    ow = conv_trans_out_dim(wd, s, pw, sw, dw, opw)
    y = np.empty((n, oh, ow, c), dtype=x.dtype)
    rc = getattr(lib(), "oracle_conv_trans_" + t)(_p(x), _p(w), _p(y), n, h, wd, f, r, s, c,
                                                  ph, pw, sh, sw, dh, dw, oh, ow)
    return None if rc else y


def g2bmm(A, B, width, dilation=1):
    """C[b,m,j] = sum_k A[b,m,k] B[b, m + d (j - w), k]; A, B [bs,m,k] -> [bs,m,2w+1]."""
    A, B = _c(A), _c(B)
    t = _tier(A, B)
    bs, m, k = A.shape
    assert B.shape == A.shape
    C = np.empty((bs, m, 2 * width + 1), dtype=A.dtype)
    getattr(lib(), "oracle_g2bmm_" + t)(_p(A), _p(B), _p(C), bs, m, k, int(width), int(dilation))
    return C


def gbmml(A, B, dilation=1):
    """C[b,m,n] = sum_j A[b,m,j] B[b, m + d j - d w, n]; A [bs,m,2w+1], B [bs,m,n]."""
    A, B = _c(A), _c(B)
    t = _tier(A, B)
    bs, m, band = A.shape
    assert band % 2 == 1 and B.shape[:2] == (bs, m)
    n = B.shape[2]
    C = np.empty((bs, m, n), dtype=A.dtype)
    getattr(lib(), "oracle_gbmml_" + t)(_p(A), _p(B), _p(C), bs, m, (band - 1) // 2, n,
                                        int(dilation))
    return C


def transpose(x, split, after, factor=2):
    """TransposeOp(input, split, after, factor)::compute."""
    x = _c(x)
    t = _tier(x)
    prm = transpose_params(list(x.shape), split, after, factor)
    if prm is None:
        return None
    flat, aft, out = prm
    y = np.empty(out, dtype=x.dtype)
    rc = getattr(lib(), "oracle_transpose_" + t)(_p(x), _p(y), _ints(flat),
                                                 _ints(aft), len(flat))
    return None if rc else y


def permute_flat(x, flat, perm):
    """The flat form: view x as ``flat`` dims, permute by ``perm``."""
    x = _c(x)
    t = _tier(x)
    y = np.empty([flat[i] for i in perm], dtype=x.dtype)
    rc = getattr(lib(), "oracle_transpose_" + t)(_p(x), _p(y), _ints(flat),
                                                 _ints(perm), len(flat))
    return None if rc else y


def split(x, dim, sizes=None, num=None):
    x = _c(x)
    t = _tier(x)
    szs = split_sizes(x.shape[dim], sizes, num)
    if szs is None:
        return None
    outs, off = [], 0
    for s in szs:
        shp = list(x.shape)
        shp[dim] = s
        y = np.empty(shp, dtype=x.dtype)
        getattr(lib(), "oracle_split_one_" + t)(_p(x), _p(y),
                                                _ints(x.shape), x.ndim, dim,
                                                off, s)
        outs.append(y)
        off += s
    return outs


def concat(xs, dim):
    xs = [_c(x) for x in xs]
    t = _tier(*xs)
    shp = list(xs[0].shape)
    shp[dim] = sum(x.shape[dim] for x in xs)
    y = np.empty(shp, dtype=xs[0].dtype)
    off = 0
    for x in xs:
        getattr(lib(), "oracle_concat_one_" + t)(_p(x), _p(y), _ints(shp),
                                                 len(shp), dim, off,
                                                 x.shape[dim])
        off += x.shape[dim]
    return y


def pad(x, begin, end):
    x = _c(x)
    t = _tier(x)
    shp = [d + b + e for d, b, e in zip(x.shape, begin, end)]
    y = np.empty(shp, dtype=x.dtype)
    rc = getattr(lib(), "oracle_pad_" + t)(_p(x), _p(y), _ints(x.shape),
                                           _ints(begin), _ints(end), x.ndim)
    return None if rc else y


def slice_(x, begin, end):
    x = _c(x)
    t = _tier(x)
    shp = [d - b - e for d, b, e in zip(x.shape, begin, end)]
    if min(shp) < 0:
        return None
    y = np.empty(shp, dtype=x.dtype)
    rc = getattr(lib(), "oracle_slice_" + t)(_p(x), _p(y), _ints(x.shape),
                                             _ints(begin), _ints(end), x.ndim)
    return None if rc else y


def extend(x, dim, num):
    x = _c(x)
    t = _tier(x)
    shp = list(x.shape)
    shp[dim] *= num + 1
    y = np.empty(shp, dtype=x.dtype)
    getattr(lib(), "oracle_extend_" + t)(_p(x), _p(y), _ints(x.shape), x.ndim,
                                         dim, num)
    return y


_ELT = {"add": 0, "sub": 1, "mul": 2}


def eltwise(op, xs, out_shape):
    xs = [_c(x) for x in xs]
    t = _tier(*xs)
    y = np.empty(out_shape, dtype=xs[0].dtype)
    ptrs = (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    sizes = (ctypes.c_size_t * len(xs))(*[x.size for x in xs])
    rc = getattr(lib(), "oracle_eltwise_" + t)(_ELT[op], ptrs, sizes, len(xs),
                                               _p(y), ctypes.c_size_t(y.size))
    return None if rc else y


def pow_(x, power):
    """PowOp::compute (operator.cc:3330-3343): `power` copies multiplied up from 1."""
    x = _c(x)
    t = _tier(x)
    y = np.empty_like(x)
    getattr(lib(), "oracle_pow_" + t)(_p(x), _p(y), ctypes.c_size_t(x.size), int(power))
    return y


def div(a, b, out_shape):
    a = _c(a.astype(np.float32, copy=False))
    b = _c(b.astype(np.float32, copy=False))
    y = np.empty(out_shape, dtype=np.float32)
    lib().oracle_div_f32(_p(a), ctypes.c_size_t(a.size), _p(b), ctypes.c_size_t(b.size),
                         _p(y), ctypes.c_size_t(y.size))
    return y


def batchnorm(x, scale, bias, mean, var, eps=1e-5):
    """BatchNormOp::compute (operator.cc:2660-2681); channel axis 1."""
    x = _c(x.astype(np.float32, copy=False))
    ch = x.shape[1]
    inner = int(np.prod(x.shape[2:], dtype=np.int64))
    y = np.empty_like(x)
    vs = [_c(v.astype(np.float32, copy=False)) for v in (scale, bias, mean, var)]
    lib().oracle_batchnorm_f32(_p(x), _p(vs[0]), _p(vs[1]), _p(vs[2]), _p(vs[3]), _p(y),
                               ctypes.c_size_t(x.shape[0]), ctypes.c_size_t(ch),
                               ctypes.c_size_t(inner), ctypes.c_float(eps))
    return y


def gather(x, indices, axis):
    """GatherOp (operator.cc:3420-3428, code_engine.cc:1465-1498): index dims first."""
    x = _c(x.astype(np.float32, copy=False))
    idx = _c(np.asarray(indices).astype(np.int32))
    pre = int(np.prod(x.shape[:axis], dtype=np.int64))
    post = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = np.empty(tuple(idx.shape) + x.shape[:axis] + x.shape[axis + 1:], dtype=np.float32)
    lib().oracle_gather_f32(_p(x), _p(idx), _p(y), ctypes.c_size_t(pre),
                            ctypes.c_size_t(x.shape[axis]), ctypes.c_size_t(post),
                            ctypes.c_size_t(idx.size))
    return y


def reduce_mean(x, axis):
    x = _c(x.astype(np.float32, copy=False))
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    shp = list(x.shape)
    shp[axis] = 1
    y = np.empty(shp, dtype=np.float32)
    lib().oracle_reduce_mean_f32(_p(x), _p(y), ctypes.c_size_t(outer),
                                 ctypes.c_size_t(x.shape[axis]), ctypes.c_size_t(inner))
    return y


SPLIT, REORDER, FUSE = 0, 1, 2


def trans_chain(x, micro_ops):
    """Evaluate a TransSplit/TransReorder/TransFuse chain
    (src/Transpose/transpose.cc). ``micro_ops`` is a list of
    ("split", index, in_dim, extr, copys) | ("reorder", perm) |
    ("fuse", index, pad, dels)."""
    x = _c(x)
    t = _tier(x)
    enc, perms = [], []
    for op in micro_ops:
        if op[0] == "split":
            enc += [SPLIT, op[1], op[2], op[3], op[4], 0]
        elif op[0] == "reorder":
            enc += [REORDER, 0, 0, 0, 0, 0]
            perms += list(op[1])
        elif op[0] == "fuse":
            enc += [FUSE, op[1], op[2], op[3], 0, 0]
        else:
            raise ValueError(op[0])
    out_dims = (ctypes.c_int * 8)()
    fn = getattr(lib(), "oracle_trans_chain_" + t)
    rk = fn(_p(x), None, _ints(x.shape), x.ndim, _ints(enc), len(micro_ops),
            _ints(perms), out_dims)
    if rk < 0:
        return None
    y = np.empty([out_dims[i] for i in range(rk)], dtype=x.dtype)
    fn(_p(x), _p(y), _ints(x.shape), x.ndim, _ints(enc), len(micro_ops),
       _ints(perms), out_dims)
    return y


def fastrand(n, seed=0, mod=10000):
    """Tensor::dataRand's one-thread stream, include/tensor.h:171-186, 371-374."""
    out = np.empty(n, dtype=np.uint32)
    lib().oracle_fastrand_fill(_p(out), ctypes.c_size_t(n), int(seed), int(mod))
    return out


# ------------------------------------------------- fp32-only (unpinned) pieces

ACT = {"none": 0, "relu": 1, "sigmoid": 2, "tanh": 3, "gelu": 4}


def activation(x, act):
    x = _c(x.astype(np.float32, copy=False))
    y = np.empty_like(x)
    lib().oracle_activation_f32(_p(x), _p(y), ctypes.c_size_t(x.size), ACT[act])
    return y


def bias_act(x, bias, act, ch_axis=1):
    x = _c(x.astype(np.float32, copy=False))
    outer = int(np.prod(x.shape[:ch_axis], dtype=np.int64))
    ch = x.shape[ch_axis]
    inner = int(np.prod(x.shape[ch_axis + 1:], dtype=np.int64))
    y = np.empty_like(x)
    b = None if bias is None else _p(_c(bias.astype(np.float32, copy=False)))
    lib().oracle_bias_act_f32(_p(x), b, _p(y), ctypes.c_size_t(outer),
                              ctypes.c_size_t(ch), ctypes.c_size_t(inner),
                              ACT[act])
    return y


def pool2d(x, kh, kw, ph, pw, sh, sw, dh=1, dw=1, mode="max"):
    x = _c(x.astype(np.float32, copy=False))
    n, c, h, w = x.shape
    oh = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    y = np.empty((n, c, oh, ow), dtype=np.float32)
    lib().oracle_pool2d_f32(_p(x), _p(y), n, c, h, w, kh, kw, ph, pw, sh, sw,
                            dh, dw, oh, ow, 0 if mode == "max" else 1)
    return y


def softmax(x):
    x = _c(x.astype(np.float32, copy=False))
    cols = x.shape[-1]
    y = np.empty_like(x)
    lib().oracle_softmax_f32(_p(x), _p(y), ctypes.c_size_t(x.size // cols),
                             ctypes.c_size_t(cols))
    return y


def layernorm(x, gamma, beta, eps=1e-5):
    x = _c(x.astype(np.float32, copy=False))
    cols = x.shape[-1]
    y = np.empty_like(x)
    g = None if gamma is None else _p(_c(gamma.astype(np.float32)))
    b = None if beta is None else _p(_c(beta.astype(np.float32)))
    lib().oracle_layernorm_f32(_p(x), g, b, _p(y),
                               ctypes.c_size_t(x.size // cols),
                               ctypes.c_size_t(cols), ctypes.c_float(eps))
    return y


def attention(q, k, v, heads, scale):
    """The operator sequence a fused attention launch stands for, one reference operator at
    a time: head split (Transpose), scores = Matmul(Q, K, transB), Mul by the scale, row
    Softmax, Matmul with V, head merge (Transpose + Reshape). q, k, v: [seq, heads*dh]."""
    seq, width = q.shape
    dh = width // heads

    def to_heads(t):  # [seq, heads*dh] -> [heads, seq, dh]
        return transpose(_c(t), 1, [1, 0, -1], dh)

    s = matmul(to_heads(q), to_heads(k), False, True)
    s = eltwise("mul", [s, np.full((1,), scale, dtype=np.float32)], s.shape)
    ctx = matmul(softmax(s), to_heads(v))
    return transpose(ctx, -1, [1, 0, 2]).reshape(seq, width)


def expr(code, inputs):
    """MemBoundOp: evaluate the index-expression program `code` (a list of ints, the format of
    include/pet_hip.h) at every position of the output shape in its header."""
    code = [int(c) for c in code]
    at = 2
    for _ in range(code[1]):
        at += 1 + code[at]
    shape = tuple(code[at + 1:at + 1 + code[at]])
    ins = [_c(np.asarray(a, dtype=np.float32)) for a in inputs]
    out = np.empty(shape, dtype=np.float32)
    ptrs = (ctypes.c_void_p * max(1, len(ins)))(*[a.ctypes.data for a in ins])
    rc = lib().oracle_expr_f32(_ints(code), len(code), ptrs, _p(out))
    return None if rc else out
