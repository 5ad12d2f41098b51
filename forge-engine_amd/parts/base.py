"""Interfaces of the parts a decoder is put together from.

A part knows its own sizes and constants (constructor arguments), the tensors it
needs (``param_specs``) and how to run on a step's flat batch.  It never knows
which model it is in.  Roles:

* ``Embedding``:    token ids -> float32 residual stream [T, H]
* ``Norm``:         residual stream (+ pending update) -> normalised activations
* ``Mixer``:        activations [T, H] -> update [T, H]; may use the cache
* ``FeedForward``:  activations [T, H] -> update [T, H]
* ``PositionEncoding``: what a mixer needs to encode positions
* ``Block``:        the arrangement of the above in one layer
* ``Head``:         normalised rows -> float32 logits
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView
from ..kernels import ops


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part reads from the checkpoint.

    kind: ``matrix`` (kept in the compute dtype), ``vector`` (norm weights and
    biases, widened to float32, which is exact), ``int_table`` (int32).
    ``init``: how the random-weights mode draws it: ``normal`` N(0, 0.02),
    ``norm`` 1 + N(0, 0.05), ``zeros``, ``unit`` N(0, 0.25), ``uniform`` U(0, 1), ``taps`` (a short
    convolution: N(0, 0.04) with one added to the newest tap), ``small`` N(0, 0.01), ``router``
    N(0, 0.25), ``identity`` (the identity plus N(0, 0.01)).
    """

    shape: tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"
    optional: bool = False


@dataclass
class BuildContext:
    device: torch.device
    dtype: torch.dtype  # compute dtype of activations and matrices: bfloat16 or float32


class Residual:
    """The float32 residual stream of one step with at most one update that has
    not been added yet, so that the add can be fused into the next norm.

    A design with several residual streams keeps them in ``streams`` [S, T, W] (``h`` is then only
    where their sum is put at the end): an arrangement widens the one stream of the embedding into
    S copies (``widen``), its pending update comes with the matrix that mixes the old streams into
    the new ones and each stream's share of the update (``add_mixed``), and a norm that reads
    streams (``reads_streams``) takes their sum, or any weighted sum, as its input: the last norm
    of such a model reads the plain sum."""

    def __init__(self, h: Tensor) -> None:
        self.h = h
        self.pending: Tensor | None = None
        self.streams: Tensor | None = None
        self.pending_mix: tuple[Tensor, Tensor] | None = None    # (mix [S, S] indexed [from, to], share [S])
        self.pending_norm: tuple[Tensor, float] | None = None    # (weight, eps): the update is RMS-normed before it is added
        self.in_compute_dtype: Tensor | None = None               # the stream as a norm of updates last stored it beside h (the same values)

    def add(self, update: Tensor | None) -> None:
        """Leave an update pending; None: the part has added it into the stream itself."""
        self.flush()
        self.in_compute_dtype = None
        self.pending = update

    def add_normed(self, update: Tensor, weight: Tensor, eps: float) -> None:
        """Leave ``h += update * rsqrt(mean(update^2) + eps) * weight`` pending (a norm behind a
        sublayer): the next norm's kernel applies it and normalises the new stream in one pass."""
        self.flush()
        if self.streams is not None:
            raise ValueError("a norm behind a sublayer needs a model with one residual stream")
        self.in_compute_dtype = None
        self.pending, self.pending_norm = update, (weight, float(eps))

    def take_normed(self):
        """(update, weight, eps) of a pending update that is to be normed, which the caller now applies."""
        update, (weight, eps) = self.pending, self.pending_norm
        self.pending = self.pending_norm = None
        return update, weight, eps

    def add_mixed(self, update: Tensor, mix: Tensor, share: Tensor) -> None:
        """Several streams: leave ``x_t <- sum_s mix[s, t] x_s + share[t] * update`` pending."""
        self.flush()
        self.in_compute_dtype = None
        self.pending, self.pending_mix = update, (mix, share)

    def take_pending(self):
        """(update, mix, share) of what is pending, which the caller now applies itself."""
        update, mixed = self.pending, self.pending_mix
        self.pending = self.pending_mix = None
        return (update, *(mixed or (None, None)))

    def widen(self, count: int) -> Tensor:
        """The streams [count, T, W]: at first ``count`` copies of the one stream."""
        if self.streams is None:
            self.flush()
            self.streams = self.h.unsqueeze(0).repeat(count, 1, 1)
        elif self.streams.shape[0] != count:
            raise ValueError(f"the model's layers disagree on the number of streams ({self.streams.shape[0]} and {count})")
        return self.streams

    def open(self) -> Tensor:
        """The stream with nothing pending, for a part that adds its update itself."""
        if self.streams is not None:
            raise ValueError("a part that adds into the stream itself needs a model with one stream")
        self.in_compute_dtype = None
        return self.flush()

    def stored(self, out: Tensor) -> Tensor:
        """A norm of updates has just stored the new stream in the compute dtype as well (``out``): the next
        sublayer that reads the stream itself takes that copy instead of casting the stream again."""
        self.in_compute_dtype = out
        return out

    def flush(self) -> Tensor:
        if self.pending is not None:
            if self.streams is not None:
                update, mix, share = self.take_pending()
                ops.hyper_norm(self.streams, update, mix, share, None, None, None, 0.0, None)
            elif self.pending_norm is not None:
                update, weight, eps = self.take_normed()
                ops.rmsnorm_update(self.h, update, weight, eps, None)
            else:
                ops.add_rows(self.h, self.pending)
                self.pending = None
        return self.h


class Part:
    role = ""
    # False for a part whose forward decides anything on the host from the step's
    # contents (lengths, slots): its steps are not replayed from a captured graph.
    graph_safe = True

    def __init__(self, ctx: BuildContext, prefix: str = "") -> None:
        self.ctx = ctx
        self.prefix = prefix

    def name(self, local: str) -> str:
        """The checkpoint name of one of this part's tensors; an empty ``local`` is the prefix
        itself (a design that names a part's only tensor like the part)."""
        if not local:
            return self.prefix
        return f"{self.prefix}.{local}" if self.prefix else local

    def param_specs(self) -> dict[str, ParamSpec]:
        """Checkpoint name -> spec, for every tensor this part (and its
        sub-parts) reads."""
        return {}

    def set_param(self, name: str, tensor: Tensor) -> None:
        """Receive one loaded tensor (already on the device, already in the
        dtype its kind and storage call for)."""
        raise KeyError(name)

    def finalize(self) -> None:
        """Called once after every tensor was set."""

    def kernel_libraries(self) -> set[str]:
        return set()

    def token_inputs(self) -> dict[str, int]:
        """Per-token integers that this part reads beside the positions: name -> integers a token
        (a position encoding with several axes, a token type).  A step's entries bring them
        (``StepEntry.inputs``) and the part finds them as ``batch.inputs[name]``, int32 [T, width];
        tokens whose entry brings none get their position on every axis."""
        return {}


class Embedding(Part):
    role = "embedding"

    def cache_needs(self) -> CacheNeeds:
        """Fixed-size state per request that the embedding keeps between steps (none by default);
        an embedding that asks for some gets ``cache=`` (a ``CacheView`` with its states)."""
        return CacheNeeds()

    def forward(self, batch, cache: CacheView | None = None) -> Residual:
        raise NotImplementedError


class Norm(Part):
    role = "norm"

    def forward(self, residual: Residual, rows: Tensor | None = None) -> Tensor:
        """Add the pending update into the stream and return the normalised
        activations (of the rows listed, if given) in the compute dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    role = "position"

    def rotary(self) -> tuple[Tensor, int] | None:
        """(inv_freq float32 [rotary_dim / 2], rotary_dim) for mixers that rotate
        q and k, or None."""
        return None

    def magnitude(self) -> float:
        """A factor on every cosine and sine of the rotation (1: a plain rotation)."""
        return 1.0


class Mixer(Part):
    role = "mixer"
    # True for a part whose forward takes ``stream=`` (the float32 residual stream, nothing pending):
    # it may add its update into the stream itself, where its last product can do so for free, and
    # then returns None instead of the update.
    takes_stream = False

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(self, x: Tensor, batch, cache: CacheView | None, writes_cache: bool = True) -> Tensor | None:
        raise NotImplementedError


class FeedForward(Part):
    role = "feed_forward"
    takes_stream = False   # as for a mixer

    def forward(self, x: Tensor, batch) -> Tensor | None:
        raise NotImplementedError


class Head(Part):
    role = "head"

    def forward(self, z: Tensor) -> Tensor:
        raise NotImplementedError


class Block(Part):
    role = "block"

    def __init__(self, ctx: BuildContext, mixer: Mixer, feed_forward: FeedForward | None,
                 norms: dict[str, Norm], prefix: str = "") -> None:
        """``feed_forward`` None: a layer without one.  ``prefix``: where tensors of the
        arrangement itself live (most arrangements have none)."""
        super().__init__(ctx, prefix)
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def children(self) -> list[Part]:
        """The arrangement itself (it may own tensors) and the parts it arranges."""
        found: list[Part] = [self, self.mixer]
        if self.feed_forward is not None:
            found.append(self.feed_forward)
        return [*found, *self.norms.values()]

    def cache_needs(self) -> CacheNeeds:
        """What one call of the layer asks of the cache: the mixer's needs, and whatever
        fixed-size state the arrangement keeps itself (by names that the mixer does not use)."""
        return self.mixer.cache_needs()

    def forward(self, residual: Residual, batch, cache: CacheView | None, writes_cache: bool = True) -> None:
        raise NotImplementedError


def build_part(role: str, spec, ctx: BuildContext, **extra: Any) -> Part:
    """Instantiate the registered class for ``spec.kind`` with the spec's
    parameters."""
    from ..registry import part_class

    return part_class(role, spec.kind)(ctx, spec.prefix, **spec.params, **extra)
