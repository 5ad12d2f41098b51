"""Configuration of the Dubizen decoder, from its config.json keys.

config.json names the design under ``architecture`` and gives the vocabulary (``vocab``), the model
width (``width``), the norms' epsilon (``norm.eps``), the factor on every normed sublayer output
(``residual_mult``) and the list ``layers``.  Each layer entry has a ``type`` (which mixer:
``attention`` or ``latent_attention``), the mixer's sizes and constants (``mixer``) and its
feed-forward (``mlp``, or null for none).

``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``mask.size`` (the sliding
window; absent: every earlier token is seen) and ``bias_max`` (the distance at which the table of biases by distance reaches its last
row; the table's rows are the tensor's).  ``latent_attention``: ``heads``, ``dim``, ``rot_dim``,
``vdim``, ``q_rank``, ``kv_rank``, ``scale``, ``rot.dims``, ``rot.base`` and optionally ``kv_from``
(an earlier layer with a down-projection of its own and the same ``kv_rank``, ``rot_dim`` and
rotation, whose cache this layer reads).  ``mlp``: ``kind`` ``dense`` with ``ff``; or ``kind``
``moe`` with ``router.experts``, ``router.top``, ``router.scale``, optionally ``router.groups``
(``count``, ``keep``), ``expert.ff`` and optionally ``shared.ff``.  The rows of a layer's table of
biases by distance are nowhere in config.json: the checkpoint's tensor shapes give them
(``with_tensor_shapes``), or ``mixer.bias_rows`` for a model without a checkpoint; a ``q_rank`` that
config.json leaves out is read from the shapes as well.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, replace
from typing import Any, ClassVar

from .model import ConfigError, KeyReader, ModelConfig

MIXER_TYPES = ("attention", "latent_attention")
MLP_KINDS = ("dense", "moe")
DEFAULT_BIAS_ROWS = 32


def _section(raw: dict, key: str, where: str) -> dict:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where} needs an object '{key}'")
    return value


def _check_attention(raw: dict, where: str) -> None:
    read = KeyReader(raw)
    heads, kv_heads = read.integer("heads"), read.integer("kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
    read.integer("dim")
    read.integer("vdim")
    read.number("scale")
    read.number("bias_max")
    if raw.get("mask") is not None:         # without it every earlier token is seen
        KeyReader(_section(raw, "mask", where)).integer("size")
    if raw.get("bias_rows") is not None:
        read.integer("bias_rows", minimum=2)


def _check_latent(raw: dict, where: str, index: int, layers: list) -> None:
    read = KeyReader(raw)
    for key in ("heads", "dim", "vdim", "kv_rank"):
        read.integer(key)
    if raw.get("q_rank") is not None:       # else the checkpoint's tensor shapes give it
        read.integer("q_rank")
    rot_dim = read.integer("rot_dim", minimum=2)
    read.number("scale")
    rot = _section(raw, "rot", where)
    dims = KeyReader(rot).integer("dims", minimum=2)
    KeyReader(rot).number("base")
    if dims % 2 or dims > rot_dim:
        raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most rot_dim ({rot_dim})")
    source = raw.get("kv_from")
    if source is None:
        return
    if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
        raise ConfigError(f"{where}: kv_from must name an earlier layer, got {source!r}")
    other = layers[source] if isinstance(layers[source], dict) else {}
    sizes = other.get("mixer")
    if other.get("type") != "latent_attention" or not isinstance(sizes, dict) or sizes.get("kv_from") is not None:
        raise ConfigError(f"{where}: layer {source} has no latent cache of its own to read")
    for key in ("kv_rank", "rot_dim", "rot"):
        if sizes.get(key) != raw.get(key):
            raise ConfigError(f"{where}: '{key}' differs from layer {source}, whose cache it reads")


def _check_mlp(mlp: Any, where: str) -> None:
    if mlp is None:
        return
    if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
        raise ConfigError(f"{where}: mlp must be null or of kind {' / '.join(MLP_KINDS)}")
    if mlp["kind"] == "dense":
        KeyReader(mlp).integer("ff")
        return
    KeyReader(_section(mlp, "expert", where)).integer("ff")
    router = _section(mlp, "router", where)
    experts, top = KeyReader(router).integer("experts"), KeyReader(router).integer("top")
    KeyReader(router).number("scale", 1.0)
    count, keep = 1, 1
    if router.get("groups") is not None:
        groups = KeyReader(_section(router, "groups", where))
        count, keep = groups.integer("count"), groups.integer("keep")
    if experts % count or keep > count:
        raise ConfigError(f"{where}: {experts} experts do not form {count} equal groups of which {keep} are kept")
    if top > experts // count * keep:
        raise ConfigError(f"{where}: router.top ({top}) exceeds the experts of the kept groups ({experts // count * keep})")
    if mlp.get("shared") is not None:
        KeyReader(_section(mlp, "shared", where)).integer("ff")


@dataclass(frozen=True)
class DubizenConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers_json: str                  # the list ``layers`` as JSON text (a frozen, hashable form)
    eos_token_id: int | None = None

    architecture: ClassVar[str] = "Dubizen"

    @property
    def layers(self) -> list[dict]:
        return json.loads(self.layers_json)

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "DubizenConfig":
        read = KeyReader(raw)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json must list the model's layers under 'layers'")
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where} must be an object")
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXER_TYPES)})")
            mixer = _section(layer, "mixer", where)
            if kind == "attention":
                _check_attention(mixer, f"{where}.mixer")
            else:
                _check_latent(mixer, f"{where}.mixer", index, layers)
            _check_mlp(layer.get("mlp"), f"{where}.mlp")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer, got {eos!r}")
        return cls(vocab=read.integer("vocab"), width=read.integer("width"),
                   norm_eps=KeyReader(_section(raw, "norm", "config.json")).number("eps"),
                   residual_mult=read.number("residual_mult", 1.0),
                   layers_json=json.dumps(layers, sort_keys=True), eos_token_id=eos)

    def with_tensor_shapes(self, shapes: dict[str, tuple[int, ...]]) -> "DubizenConfig":
        """The rows of every layer's table of biases by distance (and a query bottleneck's width that
        config.json does not give), from the checkpoint's tensor shapes."""
        layers = self.layers
        for index, layer in enumerate(layers):
            shape = shapes.get(f"l{index}.mix.rel")
            if layer["type"] == "attention" and shape is not None and len(shape) == 2:
                layer["mixer"]["bias_rows"] = int(shape[0])
            shape = shapes.get(f"l{index}.mix.dq")
            if layer["type"] == "latent_attention" and layer["mixer"].get("q_rank") is None and shape is not None and len(shape) == 2:
                layer["mixer"]["q_rank"] = int(shape[0])
        return replace(self, layers_json=json.dumps(layers, sort_keys=True))

    def to_dict(self) -> dict[str, Any]:
        data = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "layers": self.layers}
        if self.eos_token_id is not None:
            data["eos_token_id"] = self.eos_token_id
        return data
