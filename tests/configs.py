"""Test-side view of the configuration programs: everything from
``pet_amd.programs`` plus ``OracleNS``, the same operator namespace on numpy
arrays backed by the CPU oracle."""
import numpy as np

from pet_amd.programs import *  # noqa: F401,F403
from pet_amd.programs import GpuNS  # noqa: F401


class OracleNS:
    """numpy + CPU oracle."""

    def __init__(self):
        import oracle
        self.o = oracle

    def tensor(self, a):
        return np.ascontiguousarray(a, dtype=np.float32)

    def numpy(self, t):
        return t

    def _tail(self, y, bias, act, residual, ch_axis=1):
        """bias, then the residual Add, then the activation: operator by operator."""
        if bias is not None:
            y = self.o.bias_act(y, bias, "none", ch_axis=ch_axis)
        if residual is not None:
            y = self.o.eltwise("add", [y, residual.reshape(y.shape)], y.shape)
        return self.o.activation(y, act) if act != "none" else y

    def conv2d(self, x, w, ph, pw, sh=1, sw=1, dh=1, dw=1, bias=None, act="none", residual=None):
        return self._tail(self.o.conv2d(x, w, ph, pw, sh, sw, dh, dw), bias, act, residual)

    def conv3d(self, x, w, pad, stride=(1, 1, 1), dil=(1, 1, 1), bias=None, act="none",
               residual=None):
        return self._tail(self.o.conv3d(x, w, pad, stride, dil), bias, act, residual)

    def matmul(self, A, B, transA=False, transB=False, bias=None, act="none", residual=None):
        return self._tail(self.o.matmul(A, B, transA, transB), bias, act, residual, ch_axis=2)

    def matmul_shared_lhs(self, x, W, bias=None):
        """Extend -> BatchMatmul -> Split -> bias Add per slab -> (slabs side by side)."""
        y = self.o.matmul(self.o.extend(x, 0, W.shape[0] - 1), W)
        if bias is not None:
            y = np.stack([self.o.eltwise("add", [y[i], bias[i]], y[i].shape)
                          for i in range(W.shape[0])])
        return y

    def attention(self, q, k, v, heads, scale):
        seq, hidden = q.shape[-2], q.shape[-1]
        out = self.o.attention(q.reshape(seq, hidden), k.reshape(seq, hidden),
                               v.reshape(seq, hidden), heads, float(scale.reshape(-1)[0]))
        return out.reshape(1, seq, hidden)

    def expr(self, code, inputs):
        return self.o.expr(code, inputs)

    def permute_flat(self, x, flat, perm):
        return self.o.permute_flat(x, flat, perm)

    def transpose(self, x, split, after, factor=2):
        return self.o.transpose(x, split, after, factor)

    def trans_chain(self, x, chain):
        return self.o.trans_chain(x, chain)

    def split(self, x, dim, sizes=None, num=None):
        return self.o.split(x, dim, sizes, num)

    def concat(self, xs, dim):
        return self.o.concat(xs, dim)

    def pad(self, x, b, e):
        return self.o.pad(x, b, e)

    def slice(self, x, b, e):
        return self.o.slice_(x, b, e)

    def extend(self, x, dim, num):
        return self.o.extend(x, dim, num)

    def add(self, xs, shape=None):
        return self.o.eltwise("add", xs, shape or xs[0].shape)

    def mul(self, xs, shape=None):
        return self.o.eltwise("mul", xs, shape or xs[0].shape)

    def act(self, x, act):
        return self.o.activation(x, act)

    def pool2d(self, x, kh, kw, ph, pw, sh, sw, mode="max"):
        return self.o.pool2d(x, kh, kw, ph, pw, sh, sw, mode=mode)

    def softmax(self, x):
        return self.o.softmax(x)

    def layernorm(self, x, g, b):
        return self.o.layernorm(x, g, b)

    def reshape(self, x, shape):
        return x.reshape(shape)
