"""Malusun as a plan over the generic parts.

Embedding ``embed`` times ``embedding.scale``; layers ``l<i>`` in the order config.json lists them,
each with a norm before and a norm behind both sublayers (``l<i>.norm1`` / ``norm1b`` around the
mixer, ``norm2`` / ``norm2b`` around the feed-forward; RMS norms whose weights are stored around
zero), a mixer under ``l<i>.mix`` and a feed-forward under ``l<i>.mlp`` (or none); last norm
``final.norm``; head ``head``.

Mixers by layer type: ``mamba1`` is the selective scan with its short convolution; ``attention`` is
grouped-query attention over a sliding window with a partial rotation; ``attention_2`` has biases on
q, k and v, no rotation, a penalty on distance with a slope per head (``2^(-8 (h + 1) / H)``), and a
one in the softmax's denominator.  Layers whose mixer says ``v_mix`` lean their values on those of
the first such layer (``.vmix`` is the blend's scalar).  Feed-forwards: ``dense`` is ``down(relu(up
x)^2)``; ``moe`` routes by sigmoid scores, the chosen experts' scores scale their inputs, gated SiLU
experts, beside a shared expert.
"""

from __future__ import annotations

from ..config.malusun import MalusunConfig
from ..parts.plan import LayerCall, LayerSpec, ModelPlan, PartSpec
from ..registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                   "value_mix": "vmix"}
EXPERT_NAMES = {"expert": "e{e}", "shared": "shared", "router": "router", "gate": "gate", "up": "up", "down": "down"}
DISTANCE_SLOPE_BITS = 8.0      # head h of H: slope 2^(-8 (h + 1) / H)


def _mixer(config: MalusunConfig, kind: str, sizes: dict, prefix: str, value_mix: str | None) -> PartSpec:
    width = config.width
    if kind == "mamba1":
        return PartSpec("selective_scan", {"hidden_size": width, "inner": sizes["inner"], "state": sizes["state"],
                                           "dt_rank": sizes["dt_rank"], "conv_taps": sizes["conv"]}, prefix)
    params = {"hidden_size": width, "num_heads": sizes["heads"], "num_kv_heads": sizes["kv_heads"], "head_dim": sizes["dim"],
              "value_dim": sizes["vdim"], "scale": sizes["scale"], "window": (sizes.get("mask") or {}).get("size"), "value_mix": value_mix,
              "names": ATTENTION_NAMES, "force_general": True}
    if kind == "attention":
        rot = sizes["rot"]
        params["position"] = PartSpec("rotary", {"head_dim": sizes["dim"], "theta": rot["base"], "rotary_dim": rot["dims"],
                                                 "precise": True})
    else:
        params.update(position=PartSpec("none"), bias=True, output_bias=False, bias_init="small", fixed_sink=0.0,
                      distance_slope_bits=DISTANCE_SLOPE_BITS)
    return PartSpec("gqa_attention", params, prefix)


def _feed_forward(config: MalusunConfig, mlp: dict | None, prefix: str) -> PartSpec | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("activated_mlp", {"hidden_size": config.width, "intermediate_size": mlp["ff"],
                                          "activation": "relu_squared"}, prefix)
    shared = mlp.get("shared")
    return PartSpec("routed_experts", {
        "hidden_size": config.width, "experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
        "intermediate_size": mlp["expert"]["ff"], "shared_size": None if shared is None else shared["ff"],
        "scoring": "sigmoid", "form": "silu", "weight_input": True, "router_bias": False, "names": EXPERT_NAMES,
    }, prefix)


def malusun_plan(config: MalusunConfig) -> ModelPlan:
    width, eps = config.width, config.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"size": width, "eps": eps, "leaf": "", "offset": 1.0}, name)

    layers, unread, mixing_seen = [], set(), False
    for index, layer in enumerate(config.layers):
        prefix = f"l{index}"
        value_mix = None
        if layer["type"] != "mamba1" and layer["mixer"].get("v_mix"):
            value_mix = "blend" if mixing_seen else "source"
            mixing_seen = True
        feed_forward = _feed_forward(config, layer.get("mlp"), f"{prefix}.mlp")
        norms = {"input": norm(f"{prefix}.norm1"), "mixer_out": norm(f"{prefix}.norm1b")}
        if feed_forward is not None:
            norms.update(post_mixer=norm(f"{prefix}.norm2"), ff_out=norm(f"{prefix}.norm2b"))
        else:       # a checkpoint may still hold the norms around a feed-forward that is not there
            unread |= {f"{prefix}.norm2", f"{prefix}.norm2b"}
        layers.append(LayerSpec("sandwich_norm", _mixer(config, layer["type"], layer["mixer"], f"{prefix}.mix", value_mix),
                                feed_forward, norms))
    sizes = {"vocab_size": config.vocab, "hidden_size": width, "leaf": ""}
    return ModelPlan(
        hidden_size=width,
        vocab_size=config.vocab,
        embedding=PartSpec("token_embedding", dict(sizes, scale=config.embedding_scale), "embed"),
        layers=tuple(layers),
        schedule=tuple(LayerCall(index) for index in range(len(layers))),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", dict(sizes), "head"),
        eos_token_ids=frozenset() if config.eos_token_id is None else frozenset({config.eos_token_id}),
        max_positions=None,
        ignorable_names=frozenset(unread),
    )


register_architecture(MalusunConfig.architecture, MalusunConfig, malusun_plan)
