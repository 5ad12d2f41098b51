"""Gated SiLU feed-forward: ``down(silu(gate(x)) * up(x))``, no biases
(reference: src/forge_engine/qwen3.py:210-227).  gate and up share one fused
matrix [2I, H] so that a step makes one product for both."""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, FeedForward, ParamSpec


class SwiGLU(FeedForward):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, intermediate_size: int) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up_weight: Tensor | None = None
        self.down_weight: Tensor | None = None

    def param_specs(self):
        inter, hidden = self.intermediate_size, self.hidden_size
        return {
            self.name("gate_proj.weight"): ParamSpec((inter, hidden)),
            self.name("up_proj.weight"): ParamSpec((inter, hidden)),
            self.name("down_proj.weight"): ParamSpec((hidden, inter)),
        }

    def set_param(self, name: str, tensor: Tensor) -> None:
        inter = self.intermediate_size
        if name in (self.name("gate_proj.weight"), self.name("up_proj.weight")):
            if self.gate_up_weight is None:
                self.gate_up_weight = torch.empty((2 * inter, self.hidden_size), dtype=tensor.dtype,
                                                  device=tensor.device)
            if tensor.dtype != self.gate_up_weight.dtype:
                raise ValueError(f"{name}: gate and up projections must be stored in one dtype")
            start = 0 if name == self.name("gate_proj.weight") else inter
            self.gate_up_weight[start:start + inter].copy_(tensor)
        elif name == self.name("down_proj.weight"):
            self.down_weight = tensor
        else:
            raise KeyError(name)

    takes_stream = True

    def forward(self, x: Tensor, batch=None, stream: Tensor | None = None) -> Tensor | None:
        act = ops.linear_swiglu(x, self.gate_up_weight)
        return ops.linear_update(act, self.down_weight, stream=stream)   # the update stays float32 for the residual sum

    def kernel_libraries(self):
        return {"rowwise", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide", "gemm_tile"}


class PolyNormMLP(FeedForward):
    """``down(act(up(x)))`` with the PolyNorm activation: ``a N(z) + b N(z^2) + c N(z^3) + e``, powers
    element by element, N dividing a token's vector by its root mean square (float32, epsilon
    inside the root); the four numbers a, b, c, e are a tensor of the layer."""

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, intermediate_size: int, eps: float,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.eps = float(eps)
        self.names = dict({"up": "up", "down": "down", "act": "act"}, **(names or {}))
        self.up_weight: Tensor | None = None
        self.down_weight: Tensor | None = None
        self.coefficients: Tensor | None = None

    def param_specs(self):
        inter, hidden = self.intermediate_size, self.hidden_size
        return {
            self.name(self.names["up"]): ParamSpec((inter, hidden)),
            self.name(self.names["down"]): ParamSpec((hidden, inter)),
            self.name(self.names["act"]): ParamSpec((4,), kind="vector", init="unit"),
        }

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name == self.name(self.names["up"]):
            self.up_weight = tensor
        elif name == self.name(self.names["down"]):
            self.down_weight = tensor
        elif name == self.name(self.names["act"]):
            self.coefficients = tensor
        else:
            raise KeyError(name)

    def forward(self, x: Tensor, batch=None) -> Tensor:
        z = ops.linear(x, self.up_weight)
        act = torch.empty_like(z)
        ops.polynorm(z, self.coefficients, self.eps, act)
        return ops.linear_update(act, self.down_weight)

    def kernel_libraries(self):
        return {"stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


class ActivatedMLP(FeedForward):
    """``down(act(up(x)))`` without a gate and without biases; ``activation``: ``relu_squared``
    (``max(z, 0)^2``), ``gelu`` (``0.5 z (1 + erf(z / sqrt 2))``) or ``gelu_tanh``
    (``0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))``)."""

    ACTIVATIONS = ("relu_squared", "gelu", "gelu_tanh")

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, intermediate_size: int,
                 activation: str = "relu_squared", names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"unknown activation '{activation}' (known: {', '.join(self.ACTIVATIONS)})")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation
        self.names = dict({"up": "up", "down": "down"}, **(names or {}))
        self.up_weight: Tensor | None = None
        self.down_weight: Tensor | None = None

    def param_specs(self):
        inter, hidden = self.intermediate_size, self.hidden_size
        return {self.name(self.names["up"]): ParamSpec((inter, hidden)),
                self.name(self.names["down"]): ParamSpec((hidden, inter))}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name == self.name(self.names["up"]):
            self.up_weight = tensor
        elif name == self.name(self.names["down"]):
            self.down_weight = tensor
        else:
            raise KeyError(name)

    def forward(self, x: Tensor, batch=None) -> Tensor:
        z = ops.linear(x, self.up_weight)
        act = ops.relu_squared(z) if self.activation == "relu_squared" else ops.activate(z, self.activation)
        return ops.linear_update(act, self.down_weight)

    def kernel_libraries(self):
        return {"stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


register_part("feed_forward", "activated_mlp", ActivatedMLP)
register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "polynorm_mlp", PolyNormMLP)
