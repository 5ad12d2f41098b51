"""Dubizen as a plan over the generic parts.

Embedding ``embed``; layers ``l<i>`` in the order config.json lists them.  A layer's sublayers read
the residual stream itself, and what they put out passes a layer norm with a weight and no bias
(``l<i>.norm1`` behind the mixer, ``l<i>.norm2`` behind the feed-forward) and the factor
``residual_mult`` before it is added.  Mixer under ``l<i>.mix``, feed-forward under ``l<i>.mlp`` (or
none); last norm ``final.norm`` (a layer norm as well); the head is the embedding table.

Mixers by layer type.  ``attention``: grouped-query attention over a sliding window with biases on
q, k, v and the output (``.q.b`` ...), a weighted RMS norm of every q and k head (``.q.norm``,
``.k.norm``), no rotation, and a learned bias by distance (``.rel``, rows by bucket, a column a
head).  ``latent_attention``: queries through a bottleneck (``.dq``, ``.dq.norm``, ``.uq``), one
small cached vector a token and a rotated key part all heads share (``.dkv``, ``.dkv.norm``), keys
and values per head from the vector (``.uk``, ``.uv``), ``.o``; a layer whose mixer names
``kv_from`` has no ``.dkv`` and its call in the schedule reads the cache of the layer it names.

Feed-forwards: ``dense`` is ``down(gelu(up x))`` with the erf gelu; ``moe`` scores all experts by
a softmax, chooses by score plus ``.correction`` within the best groups, weighs the chosen by their
scores over their sum times ``router.scale``, gated SiLU experts (``.e<j>.gate/up/down``), beside a
shared expert (``.shared.*``) times ``sigmoid(.shared.sg . x)``.
"""

from __future__ import annotations

from ..config.dubizen import DEFAULT_BIAS_ROWS, DubizenConfig
from ..config.model import ConfigError
from ..parts.plan import LayerCall, LayerSpec, ModelPlan, PartSpec
from ..registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "o_bias": "o.b",
                   "q_norm": "q.norm", "k_norm": "k.norm", "distance_bias": "rel"}
LATENT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o"}
EXPERT_NAMES = {"expert": "e{e}", "shared": "shared", "router": "router", "gate": "gate", "up": "up", "down": "down",
                "correction": "correction", "shared_gate": "shared.sg"}


def _mixer(config: DubizenConfig, kind: str, sizes: dict, prefix: str) -> PartSpec:
    if kind == "attention":
        return PartSpec("gqa_attention", {
            "hidden_size": config.width, "num_heads": sizes["heads"], "num_kv_heads": sizes["kv_heads"], "head_dim": sizes["dim"],
            "value_dim": sizes["vdim"], "scale": sizes["scale"], "window": (sizes.get("mask") or {}).get("size"), "bias": True, "bias_init": "small",
            "qk_norm_eps": config.norm_eps, "position": PartSpec("none"), "force_general": True, "names": ATTENTION_NAMES,
            "distance_bias": {"rows": sizes.get("bias_rows") or DEFAULT_BIAS_ROWS, "reach": sizes["bias_max"]},
        }, prefix)
    rot = sizes["rot"]
    if sizes.get("q_rank") is None:
        raise ConfigError(f"{prefix}: neither config.json nor a checkpoint's shapes give the query bottleneck's width ('q_rank')")
    return PartSpec("latent_attention", {
        "hidden_size": config.width, "num_heads": sizes["heads"], "head_dim": sizes["dim"], "rot_dim": sizes["rot_dim"],
        "value_dim": sizes["vdim"], "q_rank": sizes["q_rank"], "kv_rank": sizes["kv_rank"], "scale": sizes["scale"],
        "eps": config.norm_eps, "own_kv": sizes.get("kv_from") is None, "names": LATENT_NAMES,
        "position": PartSpec("rotary", {"head_dim": sizes["rot_dim"], "theta": rot["base"], "rotary_dim": rot["dims"], "precise": True}),
    }, prefix)


def _feed_forward(config: DubizenConfig, mlp: dict | None, prefix: str) -> PartSpec | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("activated_mlp", {"hidden_size": config.width, "intermediate_size": mlp["ff"], "activation": "gelu"}, prefix)
    router, shared = mlp["router"], mlp.get("shared")
    groups = router.get("groups") or {"count": 1, "keep": 1}
    return PartSpec("routed_experts", {
        "hidden_size": config.width, "experts": router["experts"], "top": router["top"], "intermediate_size": mlp["expert"]["ff"],
        "shared_size": None if shared is None else shared["ff"], "shared_gate": shared is not None, "scoring": "softmax_all",
        "groups": groups["count"], "keep_groups": groups["keep"], "route_scale": router.get("scale", 1.0), "form": "silu",
        "router_bias": False, "names": EXPERT_NAMES,
    }, prefix)


def dubizen_plan(config: DubizenConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps

    def behind(name: str) -> PartSpec:
        return PartSpec("layer_norm_of_update", {"size": width, "eps": eps, "leaf": "", "factor": config.residual_mult}, name)

    layers, schedule, unread = [], [], set()
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        feed_forward = _feed_forward(config, layer.get("mlp"), f"{prefix}.mlp")
        norms = {"mixer_out": behind(f"{prefix}.norm1")}
        if feed_forward is not None:
            norms["ff_out"] = behind(f"{prefix}.norm2")
        else:       # a checkpoint may still hold the norm behind a feed-forward that is not there
            unread.add(f"{prefix}.norm2")
        layers.append(LayerSpec("output_norm", _mixer(config, layer["type"], layer["mixer"], f"{prefix}.mix"), feed_forward, norms,
                                {"hidden_size": width}))
        source = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
        schedule.append(LayerCall(index) if source is None else LayerCall(index, cache=source, writes_cache=False))
    sizes = {"vocab_size": config.vocab, "hidden_size": width, "leaf": ""}
    return ModelPlan(
        hidden_size=width,
        vocab_size=config.vocab,
        embedding=PartSpec("token_embedding", dict(sizes), "embed"),
        layers=tuple(layers),
        schedule=tuple(schedule),
        final_norm=PartSpec("layer_norm", {"size": width, "eps": eps, "leaf": "", "bias_leaf": None}, "final.norm"),
        head=PartSpec("lm_head", dict(sizes, tied=True), "embed"),
        eos_token_ids=frozenset() if config.eos_token_id is None else frozenset({config.eos_token_id}),
        max_positions=None,
        ignorable_names=frozenset(unread),
    )


register_architecture(DubizenConfig.architecture, DubizenConfig, dubizen_plan)
