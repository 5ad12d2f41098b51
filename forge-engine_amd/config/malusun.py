"""Configuration of the Malusun decoder, from its config.json keys.

config.json names the design under ``architecture`` and gives the vocabulary (``vocab``), the model
width (``width``), the norms' epsilon (``norm.eps``), a factor on the embedding
(``embedding.scale``) and the list ``layers``.  Each layer entry has a ``type`` (which mixer:
``mamba1``, ``attention`` or ``attention_2``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``: ``kind`` ``dense`` with ``ff``; ``kind`` ``moe`` with ``router.experts``,
``router.top``, ``expert.ff`` and optionally ``shared.ff``; or null for none).  Mixer keys:
``mamba1``: ``inner``, ``state``, ``dt_rank``, ``conv``; both attentions: ``heads``, ``kv_heads``,
``dim``, ``vdim``, ``scale``, optionally ``mask.size`` (the sliding window) and ``v_mix``;
``attention`` also ``rot.dims`` and ``rot.base``.  Every size and constant of a model comes from
here; nothing is pinned to one checkpoint.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("mamba1", "attention", "attention_2")
MLP_KINDS = ("dense", "moe")


def _section(raw: dict, key: str, where: str) -> dict:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where} needs an object '{key}'")
    return value


def _check_scan(raw: dict, where: str) -> None:
    read = KeyReader(raw)
    read.integer("inner")
    read.integer("dt_rank")
    if read.integer("state") > 256:
        raise ConfigError(f"{where}: up to 256 states a channel")
    if read.integer("conv") > 8:
        raise ConfigError(f"{where}: a short convolution of up to 8 taps")


def _check_attention(raw: dict, where: str, rotates: bool) -> None:
    read = KeyReader(raw)
    heads, kv_heads = read.integer("heads"), read.integer("kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    dim = read.integer("dim")
    read.integer("vdim")
    read.number("scale")
    if raw.get("mask") is not None:         # without it every earlier token is seen
        KeyReader(_section(raw, "mask", where)).integer("size")
    read.boolean("v_mix", False)
    if rotates:
        rot = _section(raw, "rot", where)
        dims = KeyReader(rot).integer("dims", minimum=2)
        KeyReader(rot).number("base")
        if dims % 2 or dims > dim:
            raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most dim ({dim})")


def _check_mlp(mlp: Any, where: str) -> None:
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
        raise ConfigError(f"{where}: mlp must be null or of kind {' / '.join(MLP_KINDS)}")
    if mlp["kind"] == "dense":
        KeyReader(mlp).integer("ff")
        return
    KeyReader(_section(mlp, "expert", where)).integer("ff")
    router = KeyReader(_section(mlp, "router", where))
    experts, top = router.integer("experts"), router.integer("top")
    if top > experts:
        raise ConfigError(f"{where}: router.top ({top}) exceeds router.experts ({experts})")
    if mlp.get("shared") is not None:
        KeyReader(_section(mlp, "shared", where)).integer("ff")


@dataclass(frozen=True)
class MalusunConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers_json: str                  # the list ``layers`` as JSON text (a frozen, hashable form)
    embedding_scale: float = 1.0
    eos_token_id: int | None = None

    architecture: ClassVar[str] = "Malusun"

    @property
    def layers(self) -> list[dict]:
        return json.loads(self.layers_json)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "MalusunConfig":
        read = KeyReader(raw)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json must list the model's layers under 'layers'")
        mixed_width = None
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where} must be an object")
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
            mixer = _section(layer, "mixer", where)
            if kind == "mamba1":
                _check_scan(mixer, f"{where}.mixer")
            else:
                _check_attention(mixer, f"{where}.mixer", rotates=kind == "attention")
                if mixer.get("v_mix"):
                    width = mixer["kv_heads"] * mixer["vdim"]
                    if mixed_width not in (None, width):
                        raise ConfigError(f"{where}.mixer: layers that mix values must have values of one width "
                                          f"(kv_heads x vdim: {width} against {mixed_width})")
                    mixed_width = width
            _check_mlp(layer.get("mlp"), f"{where}.mlp")
        embedding = raw.get("embedding")
        scale = KeyReader(embedding).number("scale", 1.0) if isinstance(embedding, dict) else 1.0
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer, got {eos!r}")
        return cls(vocab=read.integer("vocab"), width=read.integer("width"),
                   norm_eps=KeyReader(_section(raw, "norm", "config.json")).number("eps"),
                   layers_json=json.dumps(layers, sort_keys=True), embedding_scale=scale, eos_token_id=eos)

    def to_dict(self) -> dict[str, Any]:
        data = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale}, "layers": self.layers}
        if self.eos_token_id is not None:
            data["eos_token_id"] = self.eos_token_id
        return data
