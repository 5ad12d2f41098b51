"""Small Malusun configurations for the tests (config.json form), model folders with random weights,
and the plain implementation's logits for them."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

import plain_malusun as plain


def scan(inner, state, dt_rank, conv):
    return "mamba1", {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def attention(heads, kv_heads, dim, vdim, window, rot_dims, *, base=10000.0, scale=0.25, v_mix=True):
    return "attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                         "mask": {"size": window}, "rot": {"dims": rot_dims, "base": base}, "v_mix": v_mix}


def attention_2(heads, kv_heads, dim, vdim, window, *, scale=0.3, v_mix=True):
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if window is not None:        # without a mask every earlier token is seen
        sizes["mask"] = {"size": window}
    return "attention_2", sizes


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(vocab, width, layers, *, eps=1e-5, scale=1.0):
    return {"architecture": "Malusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


# every mixer and both feed-forwards; groups of two and three; two chosen experts and every expert chosen;
# no shared expert in one layer; a layer without a feed-forward; the whole head rotated in one layer
SMALL_A = config(96, 48, [
    layer(scan(40, 6, 5, 4), dense(56)),
    layer(attention(4, 2, 16, 12, 9, 8, base=1000.0), moe(5, 2, 20, shared=28)),
    layer(attention_2(6, 2, 8, 12, 13), moe(3, 3, 12)),
    layer(attention(2, 2, 12, 12, 5, 12, scale=0.4), None),
], scale=0.75)
# the values that others lean on come from a layer with biases; one tap (no convolution state) and a step
# size of rank one; one kv head with wide values; a layer that mixes no values; a window of three
SMALL_B = config(130, 40, [
    layer(attention_2(4, 4, 8, 8, 6), dense(24)),
    layer(scan(24, 16, 1, 1), moe(4, 1, 16, shared=8)),
    layer(attention(2, 1, 16, 32, 40, 4, base=200.0, scale=0.5), dense(64)),
    layer(attention_2(3, 3, 10, 6, 3, v_mix=False), moe(2, 1, 24, shared=16)),
], eps=1e-6, scale=2.0)
# recurrent layers alone: no keys or values are cached at all
SMALL_C = config(64, 32, [
    layer(scan(32, 3, 2, 2), None),
    layer(scan(16, 20, 4, 3), dense(40)),
])
# attention alone, nothing mixed, keys as wide as values: no state slot is ever read; a layer without a window
SMALL_D = config(70, 24, [
    layer(attention(4, 1, 16, 16, 7, 16, v_mix=False), dense(32)),
    layer(attention_2(2, 2, 6, 6, 4, v_mix=False), None),
    layer(attention_2(2, 1, 8, 4, None, v_mix=False), dense(16)),
])
# sizes that the matrix-core attention and the grouped products' full tiles take on the GPU
MEDIUM = config(320, 256, [
    layer(scan(512, 16, 16, 4), dense(384)),
    layer(attention(4, 2, 128, 128, 80, 64), moe(6, 2, 96, shared=64)),
    layer(attention_2(8, 2, 64, 128, 48), moe(3, 1, 160, shared=128)),
    layer(attention_2(4, 2, 128, 128, 200), dense(256)),
], scale=0.5)
CONFIGS = {"A": SMALL_A, "B": SMALL_B, "C": SMALL_C, "D": SMALL_D}
BLOCK_SIZE = {"A": 4, "B": 8, "C": 2, "D": 2}


def write_model(raw: dict, seed: int, folder, change=None) -> Path:
    """A model folder with random weights; ``change(tensors)`` may edit them before they are written."""
    from forge_engine_amd.config import load_model_config
    from forge_engine_amd.weights import write_random_model

    folder = write_random_model(load_model_config(raw), seed, folder)
    if change is not None:
        path = str(Path(folder) / "model.safetensors")
        tensors = load_file(path)
        change(tensors)
        save_file({name: t.contiguous() for name, t in tensors.items()}, path, metadata={"format": "pt"})
    return folder


def folder_weights(folder) -> tuple[dict, dict]:
    folder = Path(folder)
    return json.loads((folder / "config.json").read_text()), plain.load_weights(folder)


SAFE_MARGIN = 0.02     # of sigmoid scores


class Rows(dict):
    def __init__(self):
        super().__init__()
        self.decided = set()


def plain_logits(folder, requests, only=None) -> Rows:
    """(request, position) -> logits of the plain implementation, for whole requests.  ``decided`` holds
    the rows whose routing is beyond doubt: in no layer does the token, or any token before it in its
    request, choose its experts by a margin that the roundings of bfloat16 could turn."""
    cfg, weights = folder_weights(folder)
    want = Rows()
    for request_id, tokens in requests.items():
        if only is not None and request_id not in only:
            continue
        margins = []
        logits = plain.forward(cfg, weights, tokens, margins=margins)
        narrow = torch.stack(margins).min(0).values < SAFE_MARGIN if margins else torch.zeros(len(tokens), dtype=torch.bool)
        doubtful = torch.cumsum(narrow.to(torch.int64), 0) > 0
        for position in range(len(tokens)):
            want[(request_id, position)] = logits[position]
            if not bool(doubtful[position]):
                want.decided.add((request_id, position))
    return want


def compare(got: dict, want: Rows, dtype: str, fraction: float = 0.06, float32_factor: float = 1.0) -> float:
    """Every row the engine wrote against the plain implementation's.  float32: to 1e-5 + 1e-4 of the row's
    largest logit.  bfloat16: a row whose routing is beyond doubt to a fraction of the logits' spread; of all
    rows, four in five (a token that chooses another expert than the plain implementation, by a margin within
    bfloat16's rounding, moves its own logits and, through its keys, values and state, later ones)."""
    assert got, "no logits were written"
    worst, near = 0.0, 0
    for key, row in got.items():
        expected = want[key].to(torch.float64)
        assert bool(torch.isfinite(row).all()), f"{key}: non-finite logits"
        diff = (row.to(torch.float64) - expected).abs()
        if dtype == "float32":
            bound = float32_factor * (1e-5 + 1e-4 * float(expected.abs().max()))
            assert float(diff.max()) <= bound, f"{key}: off by {float(diff.max()):.3e} (bound {bound:.3e})"
            worst = max(worst, float(diff.max()))
            continue
        spread = float(expected.max() - expected.min())
        within = float(diff.max()) <= fraction * spread
        near += within
        if key in want.decided:
            assert within, f"{key}: off by {float(diff.max()):.3e} of a spread of {spread:.3e}"
            worst = max(worst, float(diff.max()) / spread)
    if dtype != "float32":
        assert near >= 0.8 * len(got), f"only {near} of {len(got)} rows are near the plain implementation's"
    return worst
