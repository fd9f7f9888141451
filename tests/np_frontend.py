"""A float64 mirror of the tensor API the random graphs of tests/graph_fuzz.py use, with a running
error bound: every value carries how far a float32 evaluation of the same graph may be from it,
whatever order its sums are taken in.

The bound follows the arithmetic (first-order forward error analysis, unit roundoff u = 2^-24):
a product a*b may be off by |a| e_b + |b| e_a + u |ab|, a sum over n terms by the sum of its
terms' bounds plus c(n) u sum|x_i| -- the term that grows with the sum's condition number
sum|x| / |sum x| when the result is compared relatively -- with c(n) = min(n, 2 sqrt(n) + 8):
the spread of the rounding error of n additions, not its worst case n.  A select whose
condition sits within the operands' bounds of flipping may take either branch.  Two float32
evaluations of one graph (the C oracle's sequential loops, the HIP backend's trees) then differ
by at most twice the bound; tests/test_oracle_golden.py holds the oracle itself to one bound of
the float64 value.

    import np_frontend
    v, e = np_frontend.evaluate(fn, arrays)         # fn as graph_fuzz.build returns it
"""
import numpy as np

U = 2.0 ** -24


def _c(n):
    return min(float(n), 2.0 * np.sqrt(n) + 8.0)


class T:
    def __init__(self, v, e=None):
        self.v = np.asarray(v, dtype=np.float64)
        self.e = np.zeros_like(self.v) if e is None else np.broadcast_to(np.asarray(e, dtype=np.float64), self.v.shape).copy()

    # -- shape ----------------------------------------------------------------------------------
    def shape(self): return list(self.v.shape)
    def ndim(self): return self.v.ndim
    def numel(self): return int(self.v.size)
    def _both(self, f): return T(f(self.v), f(self.e))
    def permute(self, axes): return self._both(lambda a: np.transpose(a, axes))
    def contiguous(self): return self
    def reshape(self, shape): return self._both(lambda a: a.reshape(shape))
    def unsqueeze(self, axis): return self._both(lambda a: np.expand_dims(a, axis))
    def expand(self, axis, size):
        return self._both(lambda a: np.repeat(a, size, axis=axis) if a.shape[axis] == 1 else a)
    def pad(self, pads): return self._both(lambda a: np.pad(a, pads))
    def unfold(self, axes, sizes, strides, dilations):
        (ax,), (k,), (s,), (d,) = axes, sizes, strides, dilations
        assert ax == self.v.ndim - 1
        n_out = (self.v.shape[ax] - d * (k - 1) - 1) // s + 1
        idx = (np.arange(n_out) * s)[:, None] + np.arange(k)[None, :] * d
        return self._both(lambda a: a[..., idx])

    # -- elementwise ----------------------------------------------------------------------------
    def _bin(self, o, v, e): return T(v, e + U * np.abs(v))
    def __add__(self, o): return self._bin(o, self.v + o.v, self.e + o.e)
    def __sub__(self, o): return self._bin(o, self.v - o.v, self.e + o.e)
    def __mul__(self, o): return self._bin(o, self.v * o.v, np.abs(self.v) * o.e + np.abs(o.v) * self.e + self.e * o.e)
    def __truediv__(self, o):
        v = self.v / o.v
        return self._bin(o, v, (self.e + np.abs(v) * o.e) / np.maximum(np.abs(o.v) - o.e, 1e-300))
    def neg(self): return T(-self.v, self.e)
    def sqrt(self):
        v = np.sqrt(self.v)
        return T(v, self.e / (2.0 * np.sqrt(np.maximum(self.v - self.e, 1e-300))) + U * v)
    def recip(self):
        v = 1.0 / self.v
        return T(v, self.e / np.maximum(np.abs(self.v) - self.e, 1e-300) ** 2 + U * np.abs(v))
    def sin(self):
        v = np.sin(self.v)
        return T(v, self.e + 2 * U * np.maximum(np.abs(v), U))
    def exp(self):
        v = np.exp(self.v)
        return T(v, v * np.expm1(self.e) + 2 * U * v)
    def ln(self):
        v = np.log(self.v)
        return T(v, self.e / np.maximum(self.v - self.e, 1e-300) + 2 * U * np.maximum(np.abs(v), U))
    def maximum(self, o): return T(np.maximum(self.v, o.v), np.maximum(self.e, o.e))
    def minimum(self, o): return T(np.minimum(self.v, o.v), np.maximum(self.e, o.e))

    # -- comparisons and selects: (condition, may it flip within the bounds) -----------------------
    def _cmp(self, o, f):
        return (f(self.v, o.v), np.abs(self.v - o.v) <= self.e + o.e)
    def lt(self, o): return self._cmp(o, np.less)
    def le(self, o): return self._cmp(o, np.less_equal)
    def gt(self, o): return self._cmp(o, np.greater)
    def ge(self, o): return self._cmp(o, np.greater_equal)
    def where_cond(self, cond, other):
        c, unsure = cond
        return T(np.where(c, self.v, other.v), np.where(c, self.e, other.e) + unsure * np.abs(self.v - other.v))

    # -- reductions and scans ---------------------------------------------------------------------
    def sum(self, axis):
        n = self.v.shape[axis]
        v = self.v.sum(axis)
        return T(v, self.e.sum(axis) + _c(n) * U * np.abs(self.v).sum(axis) + U * np.abs(v))
    def max(self, axis): return T(self.v.max(axis), self.e.max(axis))
    def min(self, axis): return T(self.v.min(axis), self.e.max(axis))
    def cumsum(self, axis):
        n = self.v.shape[axis]
        v = np.cumsum(self.v, axis)
        return T(v, np.cumsum(self.e, axis) + _c(n) * U * np.cumsum(np.abs(self.v), axis) + U * np.abs(v))
    def cummax(self, axis): return T(np.maximum.accumulate(self.v, axis), np.maximum.accumulate(self.e, axis))


class _Tensor:
    @staticmethod
    def ones_like(t): return T(np.ones_like(t.v))
    @staticmethod
    def zeros_like(t): return T(np.zeros_like(t.v))


class _NN:
    @staticmethod
    def relu(x): return x.maximum(_Tensor.zeros_like(x))
    @staticmethod
    def sigmoid(x): return (_Tensor.ones_like(x) + x.neg().exp()).recip()
    @staticmethod
    def softmax(x, axis):
        ex = (x - x.max(axis).unsqueeze(axis).expand(axis, x.shape()[axis])).exp()
        return ex / ex.sum(axis).unsqueeze(axis).expand(axis, x.shape()[axis])
    @staticmethod
    def log_softmax(x, axis):
        sh = x - x.max(axis).unsqueeze(axis).expand(axis, x.shape()[axis])
        return sh - sh.exp().sum(axis).ln().unsqueeze(axis).expand(axis, x.shape()[axis])
    @staticmethod
    def linear(x, w, bias=None):
        a = x.unsqueeze(2)                                    # [B, K, 1]
        b = w.permute([1, 0]).unsqueeze(0)                    # [1, K, O]
        y = (T(np.broadcast_to(a.v, a.v.shape[:2] + (b.v.shape[2],)), np.broadcast_to(a.e, a.e.shape[:2] + (b.e.shape[2],))) *
             T(np.broadcast_to(b.v, (a.v.shape[0],) + b.v.shape[1:]), np.broadcast_to(b.e, (a.e.shape[0],) + b.e.shape[1:]))).sum(1)
        return y if bias is None else y + bias.unsqueeze(0)


class Frontend:
    """Stands where graph_fuzz.build expects the frontend module."""
    Tensor = _Tensor
    nn = _NN


def evaluate(fn, arrays):
    """fn built by graph_fuzz.build(seed, Frontend, ...): (float64 value, bound on a float32 evaluation's distance from it)."""
    out = fn(*[T(a) for a in arrays])
    return out.v, out.e
