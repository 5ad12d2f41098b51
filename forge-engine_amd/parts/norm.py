"""RMSNorm over the residual stream, fused with the add of the pending update.

``y = sum * rsqrt(mean(sum^2) + eps) * w`` with ``sum = h + update``
(reference: src/forge_engine/qwen3.py:99-105 and kernels/__init__.py:12-26).
The reference rounds the normalised value to the model dtype before the weight
product; here the whole expression is float32 with one rounding at the store.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Norm, ParamSpec, Residual


class RMSNorm(Norm):
    def __init__(self, ctx: BuildContext, prefix: str, *, size: int, eps: float, leaf: str = "weight",
                 offset: float = 0.0) -> None:
        """``leaf``: the weight's name behind the prefix ("": the prefix itself is the name).
        ``offset``: what the stored weight is the distance from (1: weights stored around zero,
        applied as ``1 + w``; the sum is formed once, in float32, when the tensor is loaded)."""
        super().__init__(ctx, prefix)
        self.size = size
        self.eps = float(eps)
        self.leaf = leaf
        self.offset = float(offset)
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name(self.leaf): ParamSpec((self.size,), kind="vector", init="small" if self.offset else "norm")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name(self.leaf):
            raise KeyError(name)
        self.weight = tensor + self.offset if self.offset else tensor

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if residual.pending_norm is not None:    # a norm behind the sublayer before: both norms in one pass over the row
            if rows is not None:                 # the chosen rows alone; stream and pending update are left as they are
                update, (weight, eps) = residual.pending, residual.pending_norm
                out = torch.empty((rows.numel(), self.size), dtype=self.ctx.dtype, device=residual.h.device)
                return ops.rmsnorm_update_norm(residual.h, update, weight, eps, self.weight, self.eps, out, rows=rows)
            update, weight, eps = residual.take_normed()
            out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
            return ops.rmsnorm_update_norm(residual.h, update, weight, eps, self.weight, self.eps, out)
        if rows is not None:    # the chosen rows of stream + pending update; both are left as they are
            h = residual.h
            out = torch.empty((rows.numel(), self.size), dtype=self.ctx.dtype, device=h.device)
            return ops.add_rmsnorm(h, residual.pending, self.weight, self.eps, out, rows=rows, store_sum=False)
        update, residual.pending = residual.pending, None
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return ops.add_rmsnorm(residual.h, update, self.weight, self.eps, out)

    def kernel_libraries(self):
        return {"rowwise", "stream_ops"}


class UpdateRMSNorm(RMSNorm):
    """RMSNorm of a sublayer's output instead of its input: the pending update u is normalised,
    ``u * rsqrt(mean(u^2) + eps) * w``, and added into the stream, all in float32 and in one
    kernel.  Returns the new stream in the compute dtype (what the next sublayer reads: the
    sublayers of such a layer see the stream itself)."""

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if rows is not None:
            raise ValueError("a norm of updates serves whole steps, not chosen rows")
        update, residual.pending = residual.pending, None
        if update is None:
            raise ValueError("a norm of updates needs a pending update")
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return residual.stored(ops.rmsnorm_update(residual.h, update, self.weight, self.eps, out))

    def kernel_libraries(self):
        return {"rowwise", "stream_ops"}


class LayerNorm(Norm):
    """``(x - mean) / sqrt(variance + eps) * w + b`` over a row, the variance being the mean of the
    squared deviations; float32 inside, fused with the add of the pending update like the other
    norms.  It also serves models with several residual streams (``reads_streams``): its input is
    then ``sum_s read[s] x_s`` (``read`` None: the plain sum), taken after the pending update went
    into the streams through its mixing matrix, all in the same kernel."""

    reads_streams = True

    def __init__(self, ctx: BuildContext, prefix: str, *, size: int, eps: float, leaf: str = "weight",
                 bias_leaf: str | None = "bias") -> None:
        """``leaf`` / ``bias_leaf``: the tensors' names behind the prefix ("": the prefix itself);
        ``bias_leaf`` None: a layer norm with a weight and no bias."""
        super().__init__(ctx, prefix)
        self.size = size
        self.eps = float(eps)
        self.leaf, self.bias_leaf = leaf, bias_leaf
        self.weight: Tensor | None = None
        self.bias: Tensor | None = None

    def param_specs(self):
        specs = {self.name(self.leaf): ParamSpec((self.size,), kind="vector", init="norm")}
        if self.bias_leaf is not None:
            specs[self.name(self.bias_leaf)] = ParamSpec((self.size,), kind="vector", init="small")
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name == self.name(self.leaf):
            self.weight = tensor
        elif self.bias_leaf is not None and name == self.name(self.bias_leaf):
            self.bias = tensor
        else:
            raise KeyError(name)

    def forward(self, residual: Residual, rows: Tensor | None = None, read: Tensor | None = None) -> Tensor:
        streams = residual.streams if residual.streams is not None else residual.h.unsqueeze(0)
        count = streams.shape[1] if rows is None else rows.numel()
        out = torch.empty((count, self.size), dtype=self.ctx.dtype, device=streams.device)
        if rows is not None:     # the chosen rows alone; stream and pending update are left as they are
            update, mixed = residual.pending, residual.pending_mix or (None, None)
            return ops.hyper_norm(streams, update, *mixed, read, self.weight, self.bias, self.eps, out, rows=rows, store=False)
        update, mix, share = residual.take_pending()
        return ops.hyper_norm(streams, update, mix, share, read, self.weight, self.bias, self.eps, out)

    def kernel_libraries(self):
        return {"hyper"}


class UpdateLayerNorm(Norm):
    """Layer norm (a weight, no bias) of a sublayer's output instead of its input: the pending update u
    becomes ``factor * (u - mean(u)) * rsqrt(var(u) + eps) * w`` (var: the mean of the squared deviations)
    and is added into the stream, all in float32 and in one kernel.  Returns the new stream in the compute
    dtype, which is what the next sublayer of such a layer reads."""

    def __init__(self, ctx: BuildContext, prefix: str, *, size: int, eps: float, leaf: str = "weight", factor: float = 1.0) -> None:
        super().__init__(ctx, prefix)
        self.size = size
        self.eps = float(eps)
        self.leaf = leaf
        self.factor = float(factor)
        self.weight: Tensor | None = None

    def param_specs(self):
        return {self.name(self.leaf): ParamSpec((self.size,), kind="vector", init="norm")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if name != self.name(self.leaf):
            raise KeyError(name)
        self.weight = tensor

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        if rows is not None:
            raise ValueError("a norm of updates serves whole steps, not chosen rows")
        update, residual.pending = residual.pending, None
        if update is None:
            raise ValueError("a norm of updates needs a pending update")
        out = torch.empty((residual.h.shape[0], self.size), dtype=self.ctx.dtype, device=residual.h.device)
        return residual.stored(ops.layernorm_update(residual.h, update, self.weight, self.eps, self.factor, out))

    def kernel_libraries(self):
        return {"stream_ops"}


register_part("norm", "layer_norm", LayerNorm)
register_part("norm", "layer_norm_of_update", UpdateLayerNorm)
register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "rms_norm_of_update", UpdateRMSNorm)
