"""Arrangements of a mixer, a feed-forward and norms in one layer."""

from __future__ import annotations

import dataclasses

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, FixedState
from ..kernels import ops
from ..registry import register_part
from .base import Block, BuildContext, ParamSpec, Residual


class PreNormBlock(Block):
    """``h += mixer(norm_in(h)); h += ffn(norm_post(h))`` (reference:
    src/forge_engine/qwen3.py:240-261).  Each add is left pending on the stream
    and fused into the next norm, unless the part's last product added it itself."""

    NORMS = ("input", "post_mixer")

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        x = self.norms["input"].forward(residual)
        if self.mixer.takes_stream:
            residual.add(self.mixer.forward(x, batch, cache, writes_cache, stream=residual.open()))
        else:
            residual.add(self.mixer.forward(x, batch, cache, writes_cache))
        if self.feed_forward is None:
            return
        y = self.norms["post_mixer"].forward(residual)
        if self.feed_forward.takes_stream:
            residual.add(self.feed_forward.forward(y, batch, stream=residual.open()))
        else:
            residual.add(self.feed_forward.forward(y, batch))


class OutputNormBlock(Block):
    """Norms on the sublayers' outputs only: ``h += norm_m(mixer(s)); h += norm_f(ffn(h))``.
    The sublayers read the stream itself.  With ``token_shift`` the mixer reads
    ``s_t = h_t + (h_(t-1) - h_t) * shift`` instead of ``h_t`` (element by element, h_(-1) = 0),
    where ``shift`` is a learned vector of the layer; the last h of every request is kept as
    fixed-size state, so a request may be cut into steps anywhere.  A layer may have no
    feed-forward."""

    NORMS = ("mixer_out", "ff_out")
    SHIFT_STATE = "block.shift"

    def __init__(self, ctx: BuildContext, mixer, feed_forward, norms, prefix: str = "", *,
                 hidden_size: int, token_shift: bool = False, shift_leaf: str = "shift") -> None:
        super().__init__(ctx, mixer, feed_forward, norms, prefix)
        self.hidden_size = hidden_size
        self.token_shift = token_shift
        self.shift_leaf = shift_leaf
        self.shift: Tensor | None = None

    def param_specs(self):
        if not self.token_shift:
            return {}
        return {self.name(self.shift_leaf): ParamSpec((self.hidden_size,), kind="vector", init="uniform")}

    def set_param(self, name: str, tensor: Tensor) -> None:
        if not self.token_shift or name != self.name(self.shift_leaf):
            raise KeyError(name)
        self.shift = tensor.reshape(1, self.hidden_size).contiguous()

    def cache_needs(self) -> CacheNeeds:
        needs = self.mixer.cache_needs()
        if not self.token_shift:
            return needs
        states = needs.states()
        if self.SHIFT_STATE in states:
            raise ValueError(f"the mixer's state '{self.SHIFT_STATE}' collides with the layer's own")
        states[self.SHIFT_STATE] = FixedState((self.hidden_size,), torch.float32)
        return CacheNeeds(paged=needs.paged, state=states)

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        h = residual.flush()
        if self.token_shift:
            s = ops.token_shift(h, self.shift, cache.states[self.SHIFT_STATE], batch.cu_q, batch.token_seq,
                                batch.state_slots, num_seqs=batch.num_seqs, out_dtype=self.ctx.dtype)[0]
            mixer_cache = dataclasses.replace(
                cache, states={n: t for n, t in cache.states.items() if n != self.SHIFT_STATE})
        else:       # the layer before has left the stream in the compute dtype as well, unless this is the first
            s = residual.in_compute_dtype if residual.in_compute_dtype is not None else ops.cast_rows(h, self.ctx.dtype)
            mixer_cache = cache
        residual.add(self.mixer.forward(s, batch, mixer_cache, writes_cache))
        x = self.norms["mixer_out"].forward(residual)
        if self.feed_forward is not None:
            residual.add(self.feed_forward.forward(x, batch))
            self.norms["ff_out"].forward(residual)

    def kernel_libraries(self):
        return {"stream_ops"}


class SandwichNormBlock(Block):
    """A norm before and a norm behind each sublayer: ``h += norm_mb(mixer(norm_m(h)))``, then
    ``h += norm_fb(ffn(norm_f(h)))``.  The norm behind a sublayer is left pending on the stream with
    its update (``Residual.add_normed``), so that the kernel of the next norm before a sublayer (in
    this layer, in the next one, or the model's last norm) applies both in one pass.  A layer may
    have no feed-forward."""

    NORMS = ("input", "mixer_out", "post_mixer", "ff_out")

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        x = self.norms["input"].forward(residual)
        behind = self.norms["mixer_out"]
        residual.add_normed(self.mixer.forward(x, batch, cache, writes_cache), behind.weight, behind.eps)
        if self.feed_forward is None:
            return
        y = self.norms["post_mixer"].forward(residual)
        behind = self.norms["ff_out"]
        residual.add_normed(self.feed_forward.forward(y, batch), behind.weight, behind.eps)

    def kernel_libraries(self):
        return {"stream_ops"}


class HyperConnectionBlock(Block):
    """Pre-norm sublayers over ``streams`` residual streams instead of one.  Sublayer q (the mixer,
    then the feed-forward) reads ``u = sum_s in_q[s] x_s``, computes ``y = sublayer(norm_q(u))``, and
    every stream is replaced at once, from the old ones, by ``x_t = sum_s mix_q[s, t] x_s +
    out_q[t] y``.  The tensors ``in`` [S], ``out`` [S] and ``mix`` [S, S] (indexed [from, to]) live
    under ``<prefix>.<hc1 | hc2>``.  The streams start as copies of the embedding's output and the
    model's last norm reads their sum.  The update is left pending on the stream with its matrix
    and applied inside the next norm's kernel, which forms the next sublayer's input in the same
    pass.  A layer may have no feed-forward."""

    NORMS = ("input", "post_mixer")
    SUBLAYERS = ("hc1", "hc2")

    def __init__(self, ctx: BuildContext, mixer, feed_forward, norms, prefix: str = "", *, streams: int,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, mixer, feed_forward, norms, prefix)
        if not 1 <= streams <= 8:
            raise ValueError(f"one to eight residual streams, not {streams}")
        for role, norm in norms.items():
            if not getattr(norm, "reads_streams", False):
                raise ValueError(f"the norm '{role}' of a layer with several streams must be one that reads streams")
        self.streams = streams
        self.names = dict({"in": "in", "out": "out", "mix": "mix"}, **(names or {}))
        self.sublayers = self.SUBLAYERS if feed_forward is not None else self.SUBLAYERS[:1]
        self.weights: dict[str, Tensor] = {}

    def _name(self, sublayer: str, key: str) -> str:
        return self.name(f"{sublayer}.{self.names[key]}")

    def param_specs(self):
        s = self.streams
        specs = {}
        for sublayer in self.sublayers:
            specs[self._name(sublayer, "in")] = ParamSpec((s,), kind="vector", init="uniform")
            specs[self._name(sublayer, "out")] = ParamSpec((s,), kind="vector", init="norm")
            specs[self._name(sublayer, "mix")] = ParamSpec((s, s), kind="vector", init="identity")
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        for sublayer in self.sublayers:
            for key in ("in", "out", "mix"):
                if name == self._name(sublayer, key):
                    self.weights[f"{sublayer}.{key}"] = tensor.contiguous()
                    return
        raise KeyError(name)

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        residual.widen(self.streams)
        w = self.weights
        x = self.norms["input"].forward(residual, read=w["hc1.in"])
        residual.add_mixed(self.mixer.forward(x, batch, cache, writes_cache), w["hc1.mix"], w["hc1.out"])
        if self.feed_forward is not None:
            y = self.norms["post_mixer"].forward(residual, read=w["hc2.in"])
            residual.add_mixed(self.feed_forward.forward(y, batch), w["hc2.mix"], w["hc2.out"])

    def kernel_libraries(self):
        return {"hyper"}


register_part("block", "hyper_connections", HyperConnectionBlock)
register_part("block", "pre_norm", PreNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
register_part("block", "output_norm", OutputNormBlock)
