"""A plain, slow implementation of the Malusun decoder, one function per mechanism, in float64 on
the CPU.  It shares no code with the package: the tests compare the engine with it.

Malusun: an embedding times a constant; layers with a norm before and a norm behind each sublayer
(``x += norm_b(mixer(norm_a(x)))``, then the same around the feed-forward), the norms' weights
stored around zero; three mixers (a selective-scan recurrence with a short convolution, windowed
rotary attention, windowed attention with biases, a distance penalty and one more term in the
softmax's denominator); values that lean on the first such layer's values; feed-forwards that are
dense with a squared relu or a mixture of gated experts whose router weight scales the expert's
input; a last norm and a head of its own.

A model is (config dict, {tensor name: float64 tensor}).  ``forward`` runs whole sequences;
``Stepper`` runs a request token by token from explicit state, which is what the whole-sequence
functions are checked against in the tests of this file's own.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + weight)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor, before: torch.Tensor | None = None) -> torch.Tensor:
    """x [T, C], taps [C, K] (the last column weighs the token itself), bias [C]; ``before``
    [K - 1, C]: the rows ahead of x (zeros at a sequence's start)."""
    count = taps.shape[1]
    if before is None:
        before = torch.zeros((count - 1, x.shape[1]), dtype=x.dtype)
    padded = torch.cat([before, x], dim=0)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(count):
            out[t] += taps[:, j] * padded[t + j]
    return out + bias


def selective_scan_mixer(h: torch.Tensor, w: dict, p: str, sizes: dict, state: dict | None = None) -> torch.Tensor:
    """The recurrence S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n read by C, per channel c.
    ``state`` (optional) carries 'S' [inner, n] and 'conv' [taps - 1, inner] between calls."""
    inner, n, rank = sizes["inner"], sizes["state"], sizes["dt_rank"]
    xz = h @ w[p + ".in"].T
    x_raw, z = xz[:, :inner], xz[:, inner:]
    before = None if state is None else state.get("conv")
    x = silu(causal_conv(x_raw, w[p + ".conv"], w[p + ".conv.b"], before))
    if state is not None and sizes["conv"] > 1:
        rows = torch.cat([before if before is not None else torch.zeros((sizes["conv"] - 1, inner), dtype=h.dtype), x_raw])
        state["conv"] = rows[-(sizes["conv"] - 1):].clone()
    dbc = x @ w[p + ".x"].T
    dt = softplus(dbc[:, :rank] @ w[p + ".dt"].T + w[p + ".dt.b"])
    b, c = dbc[:, rank:rank + n], dbc[:, rank + n:rank + 2 * n]
    a = -torch.exp(w[p + ".A_log"])
    s = torch.zeros((inner, n), dtype=h.dtype) if state is None or "S" not in state else state["S"]
    ys = []
    for t in range(h.shape[0]):
        s = torch.exp(dt[t][:, None] * a) * s + (dt[t] * x[t])[:, None] * b[t][None, :]
        ys.append(s @ c[t] + w[p + ".D"] * x[t])
    if state is not None:
        state["S"] = s
    y = torch.stack(ys) * silu(z)
    return y @ w[p + ".o"].T


def rotate_half_layout(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, D]: the first ``dims`` dims of every head turned, dim i paired with i + dims/2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    angle = positions.to(F64)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def distance_slopes(heads: int) -> torch.Tensor:
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=F64)


def windowed_attention(q, k, v, q_positions, k_positions, *, scale: float, window: int, slopes=None, one_more: bool = False):
    """q [Tq, H, D], k [Tk, G, D], v [Tk, G, Dv]; query at position i reads keys j with
    0 <= i - j < window; ``slopes`` [H]: slope * (i - j) comes off the score; ``one_more``: a one
    joins the softmax's denominator."""
    heads, groups = q.shape[1], k.shape[1]
    out = torch.zeros((q.shape[0], heads, v.shape[2]), dtype=q.dtype)
    for h in range(heads):
        g = h // (heads // groups)
        score = (q[:, h] @ k[:, g].T) * scale
        distance = q_positions[:, None] - k_positions[None, :]
        if slopes is not None:
            score = score - slopes[h] * distance.to(q.dtype)
        seen = (distance >= 0) & (distance < window)
        score = torch.where(seen, score, torch.full_like(score, -math.inf))
        top = torch.clamp(score.max(dim=1, keepdim=True).values, min=0.0 if one_more else -math.inf)
        e = torch.exp(score - top)
        denominator = e.sum(dim=1, keepdim=True)
        if one_more:
            denominator = denominator + torch.exp(-top)
        out[:, h] = (e / denominator) @ v[:, g]
    return out


def attention_mixer(h, w, p, sizes, positions, kind: str, shared: dict, cache: dict | None = None) -> torch.Tensor:
    """Both attention mixers.  ``shared`` passes the first value-mixing layer's values of these
    tokens on to the later ones; ``cache`` (optional) holds 'k', 'v', 'pos' of the tokens before."""
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q, k, v = h @ w[p + ".q"].T, h @ w[p + ".k"].T, h @ w[p + ".v"].T
    if kind == "attention_2":
        q, k, v = q + w[p + ".q.b"], k + w[p + ".k.b"], v + w[p + ".v.b"]
    count = h.shape[0]
    q, k, v = q.view(count, heads, dim), k.view(count, groups, dim), v.view(count, groups, vdim)
    if kind == "attention":
        rot = sizes["rot"]
        q = rotate_half_layout(q, positions, rot["dims"], rot["base"])
        k = rotate_half_layout(k, positions, rot["dims"], rot["base"])
    if sizes.get("v_mix"):
        if "v_first" in shared:
            lam = w[p + ".vmix"]
            v = (1.0 - lam) * v + lam * shared["v_first"].reshape(v.shape)    # heads side by side, if they are cut differently
        else:
            shared["v_first"] = v
    k_positions = positions
    if cache is not None:
        if "k" in cache:
            k, v = torch.cat([cache["k"], k]), torch.cat([cache["v"], v])
            k_positions = torch.cat([cache["pos"], positions])
        cache["k"], cache["v"], cache["pos"] = k, v, k_positions
    out = windowed_attention(q, k, v, positions, k_positions, scale=sizes["scale"], window=(sizes.get("mask") or {}).get("size", 1 << 40),
                             slopes=distance_slopes(heads) if kind == "attention_2" else None,
                             one_more=kind == "attention_2")
    return out.reshape(count, heads * vdim) @ w[p + ".o"].T


def dense_feed_forward(h, w, p) -> torch.Tensor:
    return torch.relu(h @ w[p + ".up"].T) ** 2 @ w[p + ".down"].T


def gated_expert(h, w, p) -> torch.Tensor:
    return (silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def expert_mixture(h, w, p, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """Sigmoid scores, the ``top`` largest chosen (lowest index among equals), the score scales
    the expert's input; a shared expert for every token."""
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    scores = torch.sigmoid(h @ w[p + ".router"].T)
    out = torch.zeros_like(h)
    gaps = []
    for t in range(h.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(scores[t, e]), e))
        gaps.append(float(scores[t, order[top - 1]] - scores[t, order[top]]) if top < experts else 1.0)
        for e in order[:top]:
            out[t] += gated_expert(scores[t, e] * h[t], w, f"{p}.e{e}")
    if margins is not None:     # per token: by how much the last chosen score leads the first one left out
        margins.append(torch.tensor(gaps, dtype=F64))
    if mlp.get("shared") is not None:
        out = out + gated_expert(h, w, p + ".shared")
    return out


def feed_forward(h, w, p, mlp: dict, margins=None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, w, p)
    return expert_mixture(h, w, p, mlp, margins)


def run_layers(config: dict, w: dict, tokens, positions, states: list | None = None, margins=None, trail: list | None = None):
    """The residual stream after the last layer; ``states``: one dict per layer for a request
    that is run in steps; ``trail`` collects the stream after every layer."""
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    shared: dict = {}
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}"
        state = None if states is None else states[index]
        h = offset_norm(x, w[p + ".norm1"], eps)
        if layer["type"] == "mamba1":
            y = selective_scan_mixer(h, w, p + ".mix", layer["mixer"], state)
        else:
            y = attention_mixer(h, w, p + ".mix", layer["mixer"], positions, layer["type"], shared, state)
        x = x + offset_norm(y, w[p + ".norm1b"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(offset_norm(x, w[p + ".norm2"], eps), w, p + ".mlp", layer["mlp"], margins)
            x = x + offset_norm(y, w[p + ".norm2b"], eps)
        if trail is not None:
            trail.append(x.clone())
    return x


def logits_of(config: dict, w: dict, x: torch.Tensor) -> torch.Tensor:
    return offset_norm(x, w["final.norm"], config["norm"]["eps"]) @ w["head"].T


def forward(config: dict, w: dict, tokens, margins=None, trail=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence from position 0."""
    positions = torch.arange(len(tokens))
    return logits_of(config, w, run_layers(config, w, tokens, positions, None, margins, trail))


class Stepper:
    """One request run in portions of any size from explicit state (keys and values kept whole:
    the window is a mask)."""

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
