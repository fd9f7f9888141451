"""Parameters and layers: host-side mirror of `crates/nn/src/layers/`
(`parameter.rs:31-214`, `linear.rs:27-110`, `conv.rs:28-130`, `pool.rs`).

A `Parameter` owns an input tensor with gradient tracking; replacing its data replaces the
tensor, as the reference does (`parameter.rs:121-150`).  Unlike the reference it can also take
a device buffer directly (`update_buffer`), which is what lets an optimizer step stay on the
GPU.  Layer initialisation is the reference's deterministic `sin(0.1 i) * sqrt(1/fan_in)`
(`linear.rs:57-68`, `conv.rs:32-41`), biases start at zero.
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence

import numpy as np

from . import nn
from .tensor import Tensor, _INPUT_BUFFER_CACHE


class ParameterError(Exception):
    pass


class Parameter:
    def __init__(self, name: str, shape: Sequence[int], data=None):
        self.name = name
        self._shape = [int(s) for s in shape]
        data = np.zeros(self.numel(), np.float32) if data is None else np.asarray(data, np.float32).ravel()
        if data.size != self.numel():
            raise ParameterError(f"Data length {data.size} doesn't match shape {self._shape} (numel={self.numel()})")
        self._initial: Optional[np.ndarray] = data.copy()     # moved to the device on first use
        self._tensor = Tensor.input(self._shape).requires_grad_(True)

    @staticmethod
    def from_data(name: str, data, shape: Sequence[int]) -> "Parameter":
        return Parameter(name, shape, data)

    def shape(self) -> List[int]:
        return list(self._shape)

    def numel(self) -> int:
        return int(np.prod(self._shape)) if self._shape else 1

    def tensor(self) -> Tensor:
        if self._initial is not None:
            self._tensor.set_data(self._initial)
            self._initial = None
        return self._tensor

    def grad(self) -> Optional[Tensor]:
        return self._tensor.grad()

    def zero_grad(self) -> None:
        self._tensor.zero_grad()

    def has_data(self) -> bool:
        return self._tensor.is_realized() or self._initial is not None

    def _replace(self) -> Tensor:
        _INPUT_BUFFER_CACHE.pop(id(self._tensor.graph), None)
        self._initial = None
        self._tensor = Tensor.input(self._shape).requires_grad_(True)
        return self._tensor

    def update_data(self, new_data) -> None:
        """New values from the host (`parameter.rs:121-150`)."""
        arr = np.asarray(new_data, np.float32).ravel()
        if arr.size != self.numel():
            raise ParameterError(f"ShapeMismatch: expected {self.numel()}, got {arr.size}")
        self._replace().set_data(arr)

    def update_buffer(self, buf) -> None:
        """New values already on the device: the buffer of a realized tensor of this shape."""
        if buf.byte_len() != 4 * self.numel():
            raise ParameterError(f"ShapeMismatch: expected {4 * self.numel()} bytes, got {buf.byte_len()}")
        self._replace().set_buffer(buf)

    def to_vec(self) -> list:
        if self._initial is not None and not self._tensor.is_realized():
            return self._initial.tolist()
        return self.tensor().to_vec()

    def to_numpy(self) -> np.ndarray:
        return np.asarray(self.to_vec(), np.float32).reshape(self._shape)


def _deterministic_init(n: int, fan_in: int) -> np.ndarray:
    bound = np.float32(math.sqrt(np.float32(1.0) / np.float32(fan_in)))
    i = np.arange(n, dtype=np.float32)
    return (np.sin(i * np.float32(0.1), dtype=np.float32) * bound).astype(np.float32)


class Linear:
    """y = x W^T + b with W [out, in] (`linear.rs:27-110`)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True):
        self.in_features, self.out_features = in_features, out_features
        self.weight = Parameter("weight", [out_features, in_features],
                                _deterministic_init(out_features * in_features, in_features))
        self.bias = Parameter("bias", [out_features]) if bias else None

    def forward(self, x: Tensor) -> Tensor:
        return nn.linear(x, self.weight.tensor(), self.bias.tensor() if self.bias else None)

    def parameters(self) -> List[Parameter]:
        return [self.weight] + ([self.bias] if self.bias else [])


class Conv2d:
    """[N,Cin,H,W] -> [N,Cout,Hout,Wout] (`conv.rs:28-130`); bias on by default here."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=(1, 1), padding=(0, 0),
                 dilation=(1, 1), bias: bool = True):
        kh, kw = kernel_size
        self.stride, self.padding, self.dilation = tuple(stride), tuple(padding), tuple(dilation)
        self.weight = Parameter("weight", [out_channels, in_channels, kh, kw],
                                _deterministic_init(out_channels * in_channels * kh * kw, in_channels * kh * kw))
        self.bias = Parameter("bias", [out_channels]) if bias else None

    def forward(self, x: Tensor) -> Tensor:
        return nn.conv2d(x, self.weight.tensor(), self.bias.tensor() if self.bias else None,
                         stride=self.stride, padding=self.padding, dilation=self.dilation)

    def parameters(self) -> List[Parameter]:
        return [self.weight] + ([self.bias] if self.bias else [])


class MaxPool2d:
    def __init__(self, kernel_size, stride=None, padding=(0, 0), dilation=(1, 1)):
        self.kernel_size, self.stride, self.padding, self.dilation = kernel_size, stride, padding, dilation

    def forward(self, x: Tensor) -> Tensor:
        return nn.max_pool2d(x, self.kernel_size, self.stride, self.padding, self.dilation)

    def parameters(self) -> List[Parameter]:
        return []
