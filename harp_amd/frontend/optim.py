"""Optimizers: mirror of `crates/nn/src/optim/` (`sgd.rs:20-110`, `adam.rs:20-120`).

The reference reads every parameter and gradient back to the host, updates `Vec<f32>`s there
and uploads the result (`optimizer.rs` `get_param_data`, `sgd.rs:73-103`); each read realizes
that gradient's graph on its own, so the forward pass runs once per parameter.  Here `step()`
builds the update as tensor graphs over the (lazy) gradients and realizes the new values of all
parameters and optimizer states as the roots of one Program: forward, backward and update run
once, on the device, and the results become the parameters' new buffers without a host copy.
The arithmetic is the reference's, in its order: `p - lr*g`; `v = mu*v - lr*g, p + v`;
Adam's `m, v, m/(1-b1^t), v/(1-b2^t), p - lr*m_hat/(sqrt(v_hat)+eps)`.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

from .layers import Parameter
from .tensor import Tensor, realize_many


class OptimError(Exception):
    pass


def _state(shape) -> Tensor:
    t = Tensor.input(shape)
    import numpy as np
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
        b1, b2 = self._betas
        c1, c2 = 1.0 - b1 ** self.t, 1.0 - b2 ** self.t
        new_p, new_m, new_v = [], [], []
        for i, (p, g) in enumerate(zip(self.params, grads)):
            if self.m[i] is None:
                self.m[i], self.v[i] = _state(p.shape()), _state(p.shape())
            m = self.m[i].scale_exact(b1) + g.scale_exact(1.0 - b1)
            v = self.v[i].scale_exact(b2) + (g * g).scale_exact(1.0 - b2)
            m_hat, v_hat = m.scale_exact(1.0 / c1), v.scale_exact(1.0 / c2)
            denom = v_hat.sqrt() + Tensor.ones_like(v_hat).scale_exact(self._eps)
            new_p.append(p.tensor() - (m_hat / denom).scale_exact(self.lr))
            new_m.append(m)
            new_v.append(v)
        realize_many(new_p + new_m + new_v + list(also))
        for p, t in zip(self.params, new_p):
            p.update_buffer(t.try_buffer())
        for i in range(len(self.params)):
            self.m[i], self.v[i] = _as_input(new_m[i]), _as_input(new_v[i])
