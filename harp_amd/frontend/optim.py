"""Optimizers: mirror of `crates/nn/src/optim/` (`sgd.rs:20-110`, `adam.rs:20-120`).

The reference reads every parameter and gradient back to the host, updates `Vec<f32>`s there
and uploads the result (`optimizer.rs` `get_param_data`, `sgd.rs:73-103`); each read realizes
that gradient's graph on its own, so the forward pass runs once per parameter.  Here `step()`
builds the update as tensor graphs over the (lazy) gradients and realizes the new values of all
parameters and optimizer states as the roots of one Program: forward, backward and update run
once, on the device, and the results become the parameters' new buffers without a host copy.
The arithmetic is the reference's, in its order: `p - lr*g`; `v = mu*v - lr*g, p + v`;
Adam's `m, v, m/(1-b1^t), v/(1-b2^t), p - (lr*m_hat)/(sqrt(v_hat)+eps)` with the bias corrections
computed in float32 by the square-and-multiply `powi` (`adam.rs:108-110`).  One difference is left:
the AST has no division node, a quotient in a graph is `x * recip(y)` (as the reference's own
tensor division is), so each of the three quotients of an Adam update may differ from the host
loop's IEEE division by one unit in the last place.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np

from .layers import Parameter
from .tensor import Tensor, realize_many


class OptimError(Exception):
    pass


def _state(shape) -> Tensor:
    t = Tensor.input(shape)
    t.set_data(np.zeros(int(np.prod(shape)) if shape else 1, np.float32))
    return t


def _as_input(t: Tensor) -> Tensor:
    """A fresh input tensor bound to the realized buffer of `t` (the next step reads it)."""
    n = Tensor.input(t.shape())
    n.set_buffer(t.try_buffer())
    return n


class _Optimizer:
    def __init__(self, params: Sequence[Parameter], lr: float):
        self.params: List[Parameter] = list(params)
        self.lr = float(lr)

    def zero_grad(self) -> None:
        for p in self.params:
            p.zero_grad()

    def learning_rate(self) -> float:
        return self.lr

    def set_learning_rate(self, lr: float) -> None:
        self.lr = float(lr)

    def _grads(self) -> List[Tensor]:
        out = []
        for p in self.params:
            g = p.grad()
            if g is None:
                raise OptimError(f"NoGradient: parameter '{p.name}' has no gradient; call backward first")
            out.append(g)
        return out


class SGD(_Optimizer):
    def __init__(self, params: Sequence[Parameter], lr: float, momentum: float = 0.0):
        super().__init__(params, lr)
        self._momentum = float(momentum)
        self.velocity: List[Optional[Tensor]] = [None] * len(self.params)

    @staticmethod
    def with_momentum(params, lr: float, momentum: float) -> "SGD":
        return SGD(params, lr, momentum)

    def momentum(self) -> float:
        return self._momentum

    def step(self, also: Sequence[Tensor] = ()) -> None:
        """Updates every parameter; tensors in `also` (the loss, say) are realized by the same
        Program, so the forward pass they share with the gradients runs once."""
        grads = self._grads()
        new_p, new_v = [], []
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if self._momentum > 0.0:
                if self.velocity[i] is None:
                    self.velocity[i] = _state(p.shape())
                v = self.velocity[i].scale_exact(self._momentum) - g.scale_exact(self.lr)
                new_v.append(v)
                new_p.append(p.tensor() + v)
            else:
                new_p.append(p.tensor() - g.scale_exact(self.lr))
        realize_many(new_p + new_v + list(also))
        for p, t in zip(self.params, new_p):
            p.update_buffer(t.try_buffer())
        for i, t in enumerate(new_v):
            self.velocity[i] = _as_input(t)


def powi_f32(base: float, exp: int) -> np.float32:
    """`f32::powi`: square-and-multiply in float32, the exponent's bits from the lowest up."""
    a, r, b = np.float32(base), np.float32(1.0), abs(int(exp))
    while True:
        if b & 1:
            r = np.float32(r * a)
        b >>= 1
        if b == 0:
            break
        a = np.float32(a * a)
    return np.float32(1.0) / r if exp < 0 else r


class Adam(_Optimizer):
    def __init__(self, params: Sequence[Parameter], lr: float, betas=(0.9, 0.999), eps: float = 1e-8):
        super().__init__(params, lr)
        self._betas, self._eps, self.t = (float(betas[0]), float(betas[1])), float(eps), 0
        self.m: List[Optional[Tensor]] = [None] * len(self.params)
        self.v: List[Optional[Tensor]] = [None] * len(self.params)

    @staticmethod
    def with_betas(params, lr: float, betas, eps: float) -> "Adam":
        return Adam(params, lr, betas, eps)

    def betas(self):
        return self._betas

    def eps(self) -> float:
        return self._eps

    def time_step(self) -> int:
        return self.t

    def step(self, also: Sequence[Tensor] = ()) -> None:
        grads = self._grads()
        self.t += 1
        b1, b2 = np.float32(self._betas[0]), np.float32(self._betas[1])
        one = np.float32(1.0)
        c1, c2 = one - powi_f32(b1, self.t), one - powi_f32(b2, self.t)
        lr, eps = np.float32(self.lr), np.float32(self._eps)

        def over(x: Tensor, c) -> Tensor:                      # x / c, the way a graph divides
            return x * Tensor.ones_like(x).scale_exact(float(c)).recip()
        new_p, new_m, new_v = [], [], []
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if self.m[i] is None:
                self.m[i], self.v[i] = _state(p.shape()), _state(p.shape())
            m = self.m[i].scale_exact(float(b1)) + g.scale_exact(float(one - b1))
            # (1 - b2) * g * g associates to the left
            v = self.v[i].scale_exact(float(b2)) + g.scale_exact(float(one - b2)) * g
            m_hat, v_hat = over(m, c1), over(v, c2)
            denom = v_hat.sqrt() + Tensor.ones_like(v_hat).scale_exact(float(eps))
            new_p.append(p.tensor() - m_hat.scale_exact(float(lr)) * denom.recip())
            new_m.append(m)
            new_v.append(v)
        realize_many(new_p + new_m + new_v + list(also))
        for p, t in zip(self.params, new_p):
            p.update_buffer(t.try_buffer())
        for i in range(len(self.params)):
            self.m[i], self.v[i] = _as_input(new_m[i]), _as_input(new_v[i])
