"""A plain, slow implementation of the Dubizen decoder, one function per mechanism, in float64 on
the CPU.  It shares no code with the package: the tests compare the engine with it.

Dubizen: layers whose sublayers read the residual stream itself and whose outputs pass a layer norm
(weight, no bias) and a constant factor before they are added, ``x += m LN(mixer(x))``, then
``x += m LN(ff(x))``.  Two mixers: grouped-query attention over a sliding window with biases, a
weighted RMS norm of every q and k head, no rotation, and a learned bias by distance (distances in
buckets: one each up to half the table, logarithmic steps beyond); and attention through a latent
(queries through a low-rank bottleneck; keys and values made per head from one small cached vector
per token, plus one rotated key part that all heads share), where a layer may read the cached
vectors of an earlier layer.  Feed-forwards: dense with the erf gelu, or softmax-scored experts
chosen within the best groups by corrected scores, beside a gated shared expert.  The head is the
embedding table.

A model is (config dict, {tensor name: float64 tensor}).  ``forward`` runs whole sequences;
``Stepper`` runs a request in portions from explicit state (keys, values, latents).
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ norms and activations

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt((centred * centred).mean(dim=-1, keepdim=True) + eps) * weight


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ positions

def distance_bucket(n: int, rows: int, reach: float) -> int:
    """Row of the bias table for distance n: one row a distance below half the table, then
    logarithmic steps that reach the last row at distance ``reach``."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (rows - half))))


def rotate(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., D]: the first ``dims`` of the last axis turn, dim i with dim i + dims / 2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    angle = positions.to(F64)[:, None] * freq[None, :]
    while angle.dim() < x.dim():
        angle = angle.unsqueeze(1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(angle) - v * torch.sin(angle), v * torch.cos(angle) + u * torch.sin(angle), x[..., dims:]], dim=-1)


# ------------------------------------------------------------------ mixers

def softmax_read(scores: torch.Tensor, visible: torch.Tensor, values: torch.Tensor) -> torch.Tensor:
    """scores [Tq, Tk], visible the same shape (bool), values [Tk, Dv]."""
    scores = scores.masked_fill(~visible, -math.inf)
    return torch.softmax(scores, dim=-1) @ values


def windowed_attention(h, w, p, sizes: dict, eps: float, positions, state: dict | None = None) -> torch.Tensor:
    heads, kv_heads, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    window, scale, reach = (sizes.get("mask") or {}).get("size"), sizes["scale"], sizes["bias_max"]     # no mask: every earlier token
    count = h.shape[0]
    q = (h @ w[p + ".q"].T + w[p + ".q.b"]).view(count, heads, dim)
    k = (h @ w[p + ".k"].T + w[p + ".k.b"]).view(count, kv_heads, dim)
    v = (h @ w[p + ".v"].T + w[p + ".v.b"]).view(count, kv_heads, vdim)
    q = rms_norm(q, w[p + ".q.norm"], eps)
    k = rms_norm(k, w[p + ".k.norm"], eps)
    key_positions = positions
    if state is not None:
        if "k" in state:
            k = torch.cat([state["k"], k])
            v = torch.cat([state["v"], v])
            key_positions = torch.cat([state["positions"], positions])
        state.update(k=k, v=v, positions=key_positions)
    table = w[p + ".rel"]
    distance = positions[:, None] - key_positions[None, :]
    visible = (distance >= 0) & (distance < (window if window is not None else distance.max() + 1))
    rows = torch.tensor([[distance_bucket(int(n), table.shape[0], reach) if n >= 0 else 0 for n in line] for line in distance.tolist()])
    out = torch.zeros((count, heads, vdim), dtype=F64)
    for head in range(heads):
        shared = head // (heads // kv_heads)
        scores = q[:, head] @ k[:, shared].T * scale + table[rows, head]
        out[:, head] = softmax_read(scores, visible, v[:, shared])
    return out.reshape(count, heads * vdim) @ w[p + ".o"].T + w[p + ".o.b"]


def latent_of(h, w, p, sizes: dict, eps: float, positions):
    """What a layer with a down-projection of its own caches per token: the normed latent and the
    rotated key part that all heads share."""
    rank, rot = sizes["kv_rank"], sizes["rot"]
    down = h @ w[p + ".dkv"].T
    latent = rms_norm(down[:, :rank], w[p + ".dkv.norm"], eps)
    return latent, rotate(down[:, rank:], positions, rot["dims"], rot["base"])


def latent_attention(h, w, p, sizes: dict, eps: float, positions, cached: tuple, key_positions) -> torch.Tensor:
    """``cached``: (latents [Tk, rank], rotated key parts [Tk, rot_dim]) of every token so far,
    this layer's own or those of the layer it reads."""
    heads, dim, rot_dim, vdim, rot = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["rot"]
    count = h.shape[0]
    q = (rms_norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps) @ w[p + ".uq"].T).view(count, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate(q[..., dim:], positions, rot["dims"], rot["base"])
    latent, key_turned = cached
    keys = (latent @ w[p + ".uk"].T).view(-1, heads, dim)
    values = (latent @ w[p + ".uv"].T).view(-1, heads, vdim)
    visible = key_positions[None, :] <= positions[:, None]
    out = torch.zeros((count, heads, vdim), dtype=F64)
    for head in range(heads):
        scores = (q_plain[:, head] @ keys[:, head].T + q_turned[:, head] @ key_turned.T) * sizes["scale"]
        out[:, head] = softmax_read(scores, visible, values[:, head])
    return out.reshape(count, heads * vdim) @ w[p + ".o"].T


# ------------------------------------------------------------------ feed-forwards

def dense_feed_forward(h, w, p) -> torch.Tensor:
    return gelu_erf(h @ w[p + ".up"].T) @ w[p + ".down"].T


def gated_expert(h, w, p) -> torch.Tensor:
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def choose_experts(scores: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """For one token: the chosen experts (best first; lowest index among equals) and the margin by
    which the last chosen leads the first one left out (among the experts that could be chosen)."""
    experts = scores.numel()
    choice = (scores + correction).tolist()
    each = experts // groups
    best = [max(choice[g * each:(g + 1) * each]) for g in range(groups)]
    kept = sorted(range(groups), key=lambda g: (-best[g], g))[:keep]
    allowed = [e for e in range(experts) if e // each in kept]
    order = sorted(allowed, key=lambda e: (-choice[e], e))
    margin = choice[order[top - 1]] - choice[order[top]] if top < len(order) else 1.0
    if keep < groups:       # a group that is nearly as good as the last kept one could turn the choice as well
        others = sorted((best[g] for g in range(groups) if g not in kept), reverse=True)
        margin = min(margin, min(best[g] for g in kept) - others[0])
    return order[:top], margin


def expert_mixture(h, w, p, mlp: dict, margins: list | None = None) -> torch.Tensor:
    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    scores = torch.softmax(h @ w[p + ".router"].T, dim=-1)
    correction = w.get(p + ".correction", torch.zeros(router["experts"], dtype=F64))
    out = torch.zeros_like(h)
    gaps = []
    for t in range(h.shape[0]):
        chosen, margin = choose_experts(scores[t], correction, router["top"], groups["count"], groups["keep"])
        gaps.append(margin)
        total = sum(scores[t, e] for e in chosen) + 1e-20
        for e in chosen:
            out[t] += scores[t, e] / total * router["scale"] * gated_expert(h[t], w, f"{p}.e{e}")
    if margins is not None:
        margins.append(torch.tensor(gaps, dtype=F64))
    if mlp.get("shared") is not None:
        out = out + torch.sigmoid(h @ w[p + ".shared.sg"].T) * gated_expert(h, w, p + ".shared")
    return out


def feed_forward(h, w, p, mlp: dict, margins=None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, w, p)
    return expert_mixture(h, w, p, mlp, margins)


# ------------------------------------------------------------------ the model

def run_layers(config: dict, w: dict, tokens, positions, states: list | None = None, margins=None, trail: list | None = None):
    """The residual stream after the last layer; ``states``: one dict per layer for a request that
    is run in steps; ``trail`` collects the stream after every layer."""
    eps, factor = config["norm"]["eps"], config["residual_mult"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kept: dict[int, tuple] = {}       # layer -> (latents, rotated key parts, their positions) of every token so far
    for index, layer in enumerate(config["layers"]):
        p, sizes = f"l{index}", layer["mixer"]
        state = None if states is None else states[index]
        if layer["type"] == "attention":
            y = windowed_attention(x, w, p + ".mix", sizes, eps, positions, state)
        else:
            source = sizes.get("kv_from")
            if source is None:
                latent, turned = latent_of(x, w, p + ".mix", sizes, eps, positions)
                key_positions = positions
                if state is not None:
                    if "latent" in state:
                        latent = torch.cat([state["latent"], latent])
                        turned = torch.cat([state["turned"], turned])
                        key_positions = torch.cat([state["positions"], positions])
                    state.update(latent=latent, turned=turned, positions=key_positions)
                kept[index] = (latent, turned, key_positions)
            latent, turned, key_positions = kept[index if source is None else source]
            y = latent_attention(x, w, p + ".mix", sizes, eps, positions, (latent, turned), key_positions)
        x = x + factor * layer_norm(y, w[p + ".norm1"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(x, w, p + ".mlp", layer["mlp"], margins)
            x = x + factor * layer_norm(y, w[p + ".norm2"], eps)
        if trail is not None:
            trail.append(x.clone())
    return x


def logits_of(config: dict, w: dict, x: torch.Tensor) -> torch.Tensor:
    return layer_norm(x, w["final.norm"], config["norm"]["eps"]) @ w["embed"].T


def forward(config: dict, w: dict, tokens, margins=None, trail=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence from position 0."""
    positions = torch.arange(len(tokens))
    return logits_of(config, w, run_layers(config, w, tokens, positions, None, margins, trail))


class Stepper:
    """One request run in portions of any size from explicit state (everything kept whole: the
    window is a mask)."""

    def __init__(self, config: dict, w: dict) -> None:
        self.config, self.w = config, w
        self.states = [{} for _ in config["layers"]]
        self.length = 0

    def step(self, tokens) -> torch.Tensor:
        positions = torch.arange(self.length, self.length + len(tokens))
        self.length += len(tokens)
        return logits_of(self.config, self.w, run_layers(self.config, self.w, tokens, positions, self.states))


def load_weights(folder) -> dict:
    """Every tensor of a model folder as float64 (integers stay integers)."""
    from pathlib import Path

    from safetensors.torch import load_file

    return {name: (t.to(F64) if t.is_floating_point() else t) for name, t in load_file(str(Path(folder) / "model.safetensors")).items()}
