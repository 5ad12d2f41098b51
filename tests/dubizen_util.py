"""Small Dubizen configurations for the tests (config.json form), model folders with random weights,
and the plain implementation's logits for them."""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import load_file, save_file

import plain_dubizen as plain


def attention(heads, kv_heads, dim, vdim, window, *, reach=20.0, rows=8, scale=0.3):
    return "attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                         "mask": {"size": window}, "bias_max": reach, "bias_rows": rows}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, *, turned=None, base=10000.0, scale=0.25, source=None):
    sizes = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
             "rot": {"dims": rot_dim if turned is None else turned, "base": base}}
    if source is not None:
        sizes["kv_from"] = source
    return "latent_attention", sizes


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None, *, groups=None, scale=1.5):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    return mlp


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def config(vocab, width, layers, *, eps=1e-5, mult=0.6):
    return {"architecture": "Dubizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}


# both mixers and both feed-forwards; a layer that reads the first layer's cache across another mixer; groups of
# two and three query heads; experts in groups of which one or two are kept; a layer without a feed-forward
SMALL_A = config(96, 48, [
    layer(latent(3, 8, 4, 6, 10, 12, base=500.0), dense(56)),
    layer(attention(4, 2, 16, 12, 9, reach=14.0, rows=6), moe(6, 2, 20, shared=28, groups=(2, 1))),
    layer(latent(2, 6, 4, 10, 7, 12, base=500.0, source=0), moe(9, 3, 12, shared=8, groups=(3, 2), scale=2.0)),
    layer(attention(6, 2, 8, 12, 13, reach=40.0, rows=10), None),
])
# the windowed layer first; a window of three and one of a single token; as many kv heads as heads; part of the
# rotated part turned; every expert of the kept groups chosen; no groups, no shared expert; a factor of one on the
# sublayers; two layers that read the same cache, and a second cache of another geometry
SMALL_B = config(130, 40, [
    layer(attention(4, 4, 8, 8, 3, reach=9.0, rows=5), dense(24)),
    layer(latent(4, 4, 8, 4, 16, 20, turned=4, base=200.0, scale=0.5), moe(4, 2, 16, groups=(2, 1))),
    layer(latent(2, 10, 8, 6, 9, 20, turned=4, base=200.0, source=1), dense(64)),
    layer(latent(5, 6, 2, 6, 12, 6, base=30.0), moe(3, 1, 24)),
    layer(latent(1, 12, 8, 16, 5, 20, turned=4, base=200.0, source=1), moe(2, 2, 8, shared=16)),
    layer(attention(2, 1, 10, 6, 1, reach=5.0, rows=4), dense(16)),
], eps=1e-6, mult=1.0)
# attention through a latent alone, one head; nothing else keeps a cache
SMALL_C = config(64, 32, [
    layer(latent(1, 16, 6, 16, 8, 10, turned=2, base=50.0), None),
    layer(latent(2, 4, 6, 4, 8, 10, turned=2, base=50.0, source=0), dense(40)),
], mult=0.25)
# windowed attention alone
SMALL_D = config(70, 24, [
    layer(attention(4, 1, 16, 16, 7, reach=100.0, rows=12), dense(32)),
    layer(attention(2, 2, 6, 6, 4, reach=3.5, rows=4), moe(4, 1, 12, shared=12, groups=(4, 2))),
], mult=1.3)
# sizes that the matrix-core kernels and the grouped products' full tiles take on the GPU
MEDIUM = config(320, 256, [
    layer(latent(4, 64, 64, 64, 96, 128, base=10000.0, scale=0.09), dense(384)),
    layer(attention(4, 2, 128, 128, 80, reach=64.0, rows=16, scale=0.09), moe(8, 2, 96, shared=64, groups=(4, 2))),
    layer(latent(6, 32, 64, 32, 64, 128, base=10000.0, scale=0.1, source=0), moe(4, 1, 160, shared=128)),
    layer(latent(16, 32, 32, 48, 128, 64, base=1000.0, scale=0.12), dense(256)),
    layer(attention(8, 2, 64, 64, 48, reach=200.0, rows=32, scale=0.12), None),
], mult=0.8)
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


SAFE_MARGIN = 0.1      # of corrected softmax scores: router logits of these models reach tens, and bfloat16 moves them by tenths


class Rows(dict):
    def __init__(self):
        super().__init__()
        self.decided = set()


def plain_logits(folder, requests, only=None) -> Rows:
    """(request, position) -> logits of the plain implementation, for whole requests.  ``decided`` holds
    the rows whose routing is beyond doubt: in no layer does the token, or any token before it in its
    request, choose its experts or their groups by a margin that the roundings of bfloat16 could turn."""
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
    bfloat16's rounding, moves its own logits and, through its keys and values, later ones)."""
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
