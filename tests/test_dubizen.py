"""Dubizen through the engine on the CPU, with the kernels' plain references patched in, against the
plain implementation (tests/plain_dubizen.py): configuration and tensor names, each mechanism alone,
and that logits do not depend on how requests are cut into steps, batched, or placed in pages and
state slots.  The kernels themselves run in the GPU tests."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import dubizen_util as du
import kernel_refs
import replay_util as ru
from forge_engine_amd.config import ConfigError, SchedulerConfig, load_model_config
from forge_engine_amd.engine import build_engine, load_model
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights.random_init import declared_tensors

plain = du.plain
F64 = torch.float64
LENGTHS = {"A": (5, 1, 14, 31), "B": (2, 9, 47, 23), "C": (7, 18, 3, 1), "D": (12, 1, 25, 6)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: du.write_model(raw, 7, tmp_path_factory.mktemp(f"dubizen_{name}")) for name, raw in du.CONFIGS.items()}


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": du.CONFIGS[name]["vocab"]}, seed, lengths)


def test_configuration_names_and_shapes(folders):
    config = load_model_config(du.SMALL_A)
    assert config.architecture == "Dubizen" and load_model_config(config.to_dict()) == config
    tensors = declared_tensors(config)
    for name, shape in {"embed": (96, 48), "final.norm": (48,), "l0.norm1": (48,), "l0.norm2": (48,), "l0.mix.dq": (10, 48),
                        "l0.mix.dq.norm": (10,), "l0.mix.uq": (36, 10), "l0.mix.dkv": (16, 48), "l0.mix.dkv.norm": (12,),
                        "l0.mix.uk": (24, 12), "l0.mix.uv": (18, 12), "l0.mix.o": (48, 18), "l0.mlp.up": (56, 48),
                        "l0.mlp.down": (48, 56), "l1.mix.q": (64, 48), "l1.mix.q.b": (64,), "l1.mix.k": (32, 48), "l1.mix.k.b": (32,),
                        "l1.mix.v": (24, 48), "l1.mix.v.b": (24,), "l1.mix.q.norm": (16,), "l1.mix.k.norm": (16,), "l1.mix.rel": (6, 4),
                        "l1.mix.o": (48, 48), "l1.mix.o.b": (48,), "l1.mlp.router": (6, 48), "l1.mlp.correction": (6,),
                        "l1.mlp.e5.gate": (20, 48), "l1.mlp.e0.down": (48, 20), "l1.mlp.shared.up": (28, 48), "l1.mlp.shared.sg": (1, 48),
                        "l2.mix.uq": (20, 7), "l2.mix.uk": (12, 12), "l2.mix.uv": (20, 12), "l2.mlp.e8.up": (12, 48),
                        "l3.mix.rel": (10, 6), "l3.norm1": (48,)}.items():
        assert tuple(tensors[name].shape) == shape, name
    # a layer that reads another's cache has no down-projection of its own; no head of its own; a layer without a
    # feed-forward has no norm behind one; a mixture without a shared expert has no gate for one
    assert not any(n in tensors for n in ("l2.mix.dkv", "l2.mix.dkv.norm", "head", "l3.norm2", "l0.mix.q.b", "l0.mix.o.b"))
    assert not any(n.startswith("l3.mlp") for n in tensors)
    assert "l3.mlp.shared.sg" not in declared_tensors(load_model_config(du.SMALL_B))
    # the rows of a table of biases come from the checkpoint's shapes
    bare = copy.deepcopy(du.SMALL_A)
    for entry in bare["layers"]:
        entry["mixer"].pop("bias_rows", None)
    shaped = load_model_config(bare).with_tensor_shapes({"l1.mix.rel": (6, 4), "l3.mix.rel": (10, 6)})
    assert tuple(declared_tensors(shaped)["l3.mix.rel"].shape) == (10, 6)
    a = du.SMALL_A
    for broken in ({**a, "layers": []},
                   {**a, "layers": [{**a["layers"][0], "type": "attention_9"}]},
                   {**a, "layers": [du.layer(du.attention(3, 2, 8, 8, 4), None)]},                  # heads no multiple of kv heads
                   {**a, "layers": [du.layer(du.attention(2, 2, 8, 8, 0), None)]},                  # an empty window
                   {**a, "layers": [du.layer(du.latent(2, 8, 4, 8, 6, 6, turned=6), None)]},        # more turned dims than the part has
                   {**a, "layers": [du.layer(du.latent(2, 8, 4, 8, 6, 6, source=0), None)]},        # reads itself
                   {**a, "layers": [a["layers"][1], du.layer(du.latent(2, 8, 4, 8, 6, 6, source=0), None)]},   # reads a windowed layer
                   {**a, "layers": [a["layers"][0], du.layer(du.latent(2, 8, 4, 8, 6, 10, base=500.0, source=0), None)]},   # another rank
                   {**a, "layers": [a["layers"][0], a["layers"][2], du.layer(du.latent(2, 8, 4, 8, 6, 12, base=500.0, source=1), None)]},  # reads a reader
                   {**a, "layers": [du.layer(du.attention(2, 2, 8, 8, 4), du.moe(6, 3, 8, groups=(3, 1)))]},    # more chosen than the kept groups hold
                   {**a, "layers": [du.layer(du.attention(2, 2, 8, 8, 4), du.moe(6, 2, 8, groups=(4, 1)))]},    # groups of unequal size
                   {**a, "layers": [du.layer(du.attention(2, 2, 8, 8, 4), {"kind": "glu", "ff": 8})]},
                   {k: v for k, v in a.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            load_model_config(broken)


def test_plain_in_steps_equals_plain_whole(folders):
    """The plain implementation's own pin: a request run from explicit state, token by token and in
    portions, gives the logits of the whole-sequence functions."""
    for name in ("A", "B", "C"):
        cfg, weights = du.folder_weights(folders[name])
        tokens = requests_of(name, 5, (29,))["r0"]
        whole = plain.forward(cfg, weights, tokens)
        for cuts in ([1] * 29, [7, 2, 13, 1, 6]):
            stepper, at = plain.Stepper(cfg, weights), 0
            for size in cuts:
                got = stepper.step(tokens[at:at + size])
                assert torch.allclose(got, whole[at:at + size], atol=1e-9), (name, at)
                at += size


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_replay_matches_plain(name, mode, folders, tmp_path, monkeypatch):
    """Whole prompts; a prompt and then token by token; portions down to two tokens; up to three
    live requests, portions beside single tokens."""
    kernel_refs.install(monkeypatch)
    requests = requests_of(name, 3, LENGTHS[name])
    trace = {"whole": ru.trace_whole, "tail": lambda r: ru.trace_tail(r, 16), "portions": ru.trace_portions,
             "mixed": lambda r: ru.trace_mixed(r, 5, max_live=3)}[mode](requests)
    got = ru.run_trace(folders[name], "float32", trace, tmp_path, block_size=du.BLOCK_SIZE[name], device="cpu", on_cpu=True)
    du.compare(got, du.plain_logits(folders[name], requests), "float32")


def test_decoding_from_the_first_token_and_far_past_every_window(folders, tmp_path, monkeypatch):
    """One token a step from position 0 on, 75 steps: every window (1, 3, 9, 13) passes over decoded tokens
    many times and the windowed layers' pages go back to the pool while the request lives."""
    kernel_refs.install(monkeypatch)
    for name in ("A", "B"):
        requests = requests_of(name, 8, (75,))
        trace = ru.trace_tail(requests, 75)
        assert len(trace.steps) == 75
        got = ru.run_trace(folders[name], "float32", trace, tmp_path / name, block_size=4, device="cpu", on_cpu=True)
        du.compare(got, du.plain_logits(folders[name], requests), "float32")


def test_pages_and_state_slots_are_used_again(folders, tmp_path, monkeypatch):
    """Seven requests through four state slots and a pool smaller than their sum: a request reads the
    rows it wrote itself, whoever held its pages before."""
    kernel_refs.install(monkeypatch)
    for name in ("A", "C"):
        requests = requests_of(name, 4, (12, 20, 7, 16, 9, 3, 11))
        trace = ru.trace_mixed(requests, 9, max_live=4)
        assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
        got = ru.run_trace(folders[name], "float32", trace, tmp_path / name, block_size=du.BLOCK_SIZE[name], device="cpu", on_cpu=True)
        du.compare(got, du.plain_logits(folders[name], requests), "float32")


def test_greedy_generation_through_the_scheduler(folders, monkeypatch):
    kernel_refs.install(monkeypatch)
    _, model = load_model(folders["A"], dtype="float32", device="cpu")
    engine = build_engine(model, scheduler_config=SchedulerConfig(block_size=4, block_capacity=64, token_budget=8, max_batch_size=3),
                          eos_token_ids=())
    prompts = list(requests_of("A", 6, (11, 4, 17)).values())
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=6)) for prompt in prompts]
    engine.run_until_idle()
    cfg, weights = du.folder_weights(folders["A"])
    for request_id, prompt in zip(ids, prompts):
        tokens = list(prompt)
        for _ in range(6):
            tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
        assert list(engine.request(request_id).output_token_ids) == tokens[len(prompt):]


# ------------------------------------------------------------------ edges and far keys, made to show

SHARP = du.config(80, 32, [
    du.layer(du.latent(2, 8, 4, 8, 12, 10, base=50.0, scale=1.0), None),
    du.layer(du.attention(2, 1, 8, 8, 6, reach=5.0, rows=6, scale=1.0), None),
    du.layer(du.latent(2, 4, 4, 6, 8, 10, base=50.0, scale=1.0, source=0), None),
    du.layer(du.attention(2, 2, 8, 8, 11, reach=30.0, rows=8, scale=1.0), None),
], mult=1.0)


def sharpen(tensors):
    """Queries and keys several times as large: the softmax of every head sits on a few keys, so one key
    that is wrongly seen, or wrongly left out, moves the result; biases by distance of order one."""
    for name in tensors:
        if name.endswith((".mix.q.norm", ".mix.uq", ".mix.dkv")):      # q and k heads of the windowed layers are normed: their norm's weight sharpens
            tensors[name] = (tensors[name].float() * 6.0).to(tensors[name].dtype)
        if name.endswith(".mix.rel"):
            tensors[name] = (tensors[name].float() * 3.0).to(tensors[name].dtype)


def test_a_window_one_token_off_a_wrong_bucket_or_a_lost_far_key_would_show(tmp_path, monkeypatch):
    """Sharp attention in portions and single tokens against the plain implementation; and the control: the
    plain implementation itself with a window one token longer or shorter, a table of biases that reaches its
    last row elsewhere, a reader that makes a cache of its own, or another first token lands far outside the
    bound."""
    kernel_refs.install(monkeypatch)
    folder = du.write_model(SHARP, 21, tmp_path / "model", change=sharpen)
    requests = {k: [t % 80 for t in v] for k, v in requests_of("A", 12, (61, 38)).items()}
    want = du.plain_logits(folder, requests)
    for mode, trace in (("portions", ru.trace_portions(requests)), ("tail", ru.trace_tail(requests, 30)),
                        ("mixed", ru.trace_mixed(requests, 3, max_live=2))):
        got = ru.run_trace(folder, "float32", trace, tmp_path / mode, block_size=4, device="cpu", on_cpu=True)
        du.compare(got, want, "float32")
    cfg, weights = du.folder_weights(folder)
    tokens = requests["r0"]
    right = plain.forward(cfg, weights, tokens)
    bound = 1e-5 + 1e-4 * float(right.abs().max())

    def moved(other_cfg, other_tokens=tokens, rows=slice(None)):
        """The largest change of any logit of the rows (a random key at an edge matters to some rows, not to all)."""
        return float((plain.forward(other_cfg, weights, other_tokens)[rows] - right[rows]).abs().max())

    for index, delta in ((1, 1), (1, -1), (3, 1), (3, -1)):
        other = copy.deepcopy(cfg)
        other["layers"][index]["mixer"]["mask"]["size"] += delta
        assert moved(other) > 100 * bound, (index, delta)
    other = copy.deepcopy(cfg)
    other["layers"][3]["mixer"]["bias_max"] = 12.0
    assert moved(other) > 100 * bound
    changed = [(tokens[0] + 1) % 80] + tokens[1:]       # attention through the latent sees the first token from the last ones
    assert moved(cfg, changed, slice(40, None)) > 5 * bound


# ------------------------------------------------------------------ each mechanism alone

def single(mixer, mlp, *, vocab=50, width=24, mult=0.5, before=None):
    layers = ([] if before is None else [before]) + [du.layer(mixer, mlp)]
    return du.config(vocab, width, layers, mult=mult)


@pytest.mark.parametrize("case", ["windowed", "windowed_one_kv_head", "no_window", "latent", "latent_reader", "dense", "experts", "experts_all"])
def test_each_mechanism_alone_through_the_engine(case, tmp_path, monkeypatch):
    """A model of one layer (two for a reader of another layer's cache) around the mechanism, in portions and
    single tokens through the engine, against the plain function for it."""
    kernel_refs.install(monkeypatch)
    quiet = du.latent(1, 4, 2, 4, 4, 4, base=10.0)
    raw = {
        "windowed": single(du.attention(6, 3, 10, 14, 5, reach=4.0, rows=4), None),
        "windowed_one_kv_head": single(du.attention(5, 1, 6, 2, 17, reach=60.0, rows=20), None),
        "no_window": single(du.attention(2, 2, 6, 10, 1, reach=11.0, rows=6), None),      # the mask is taken out below: biases up to the table's reach and beyond
        "latent": single(du.latent(3, 10, 6, 14, 9, 11, turned=4, base=77.0), None),
        "latent_reader": single(du.latent(2, 6, 6, 4, 5, 11, turned=4, base=77.0, source=0), None,
                                before=du.layer(du.latent(3, 10, 6, 14, 9, 11, turned=4, base=77.0), None)),
        "dense": single(quiet, du.dense(36)),
        "experts": single(quiet, du.moe(12, 3, 10, shared=6, groups=(4, 2), scale=2.25)),
        "experts_all": single(quiet, du.moe(3, 3, 10, scale=0.5)),
    }[case]
    if case == "no_window":
        del raw["layers"][0]["mixer"]["mask"]
    folder = du.write_model(raw, 5, tmp_path / "model")
    if case == "latent":        # a config.json that leaves the query bottleneck's width to the tensors' shapes
        import json
        stored = json.loads((folder / "config.json").read_text())
        del stored["layers"][0]["mixer"]["q_rank"]
        (folder / "config.json").write_text(json.dumps(stored))
    requests = ru.make_requests({"vocab_size": raw["vocab"]}, 2, (33, 6))
    want = du.plain_logits(folder, requests)
    for trace in (ru.trace_portions(requests, sizes=(5, 2, 9, 3)), ru.trace_tail(requests, 12)):
        got = ru.run_trace(folder, "float32", trace, tmp_path / f"out{len(trace.steps)}", block_size=4, device="cpu", on_cpu=True)
        du.compare(got, want, "float32")
    # the mechanism's own function gives what the model's layer adds
    cfg, weights = du.folder_weights(folder)
    tokens = requests["r0"]
    trail = []
    plain.forward(cfg, weights, tokens, trail=trail)
    x = weights["embed"][torch.tensor(tokens)] if len(cfg["layers"]) == 1 else trail[0]
    index = len(cfg["layers"]) - 1
    sizes, positions = cfg["layers"][index]["mixer"], torch.arange(len(tokens))
    if case.startswith("windowed"):
        y = plain.windowed_attention(x, weights, f"l{index}.mix", sizes, cfg["norm"]["eps"], positions)
    elif case.startswith("latent"):
        source = cfg["layers"][0]["mixer"]
        before = weights["embed"][torch.tensor(tokens)]
        cached = plain.latent_of(before, weights, "l0.mix", source, cfg["norm"]["eps"], positions)
        y = plain.latent_attention(x, weights, f"l{index}.mix", sizes, cfg["norm"]["eps"], positions, cached, positions)
    else:
        return
    after = x + cfg["residual_mult"] * plain.layer_norm(y, weights[f"l{index}.norm1"], cfg["norm"]["eps"])
    assert torch.allclose(after, trail[index], atol=1e-12)


def test_buckets_of_distances():
    """One row a distance below half the table, logarithmic steps beyond, the last row from the reach on;
    and the table laid out by distance, as the attention part makes it, picks the same rows."""
    from forge_engine_amd.parts.attention import GroupedQueryAttention
    from forge_engine_amd.parts.base import BuildContext
    from forge_engine_amd.parts.plan import PartSpec

    assert [plain.distance_bucket(n, 8, 16.0) for n in (0, 1, 3, 4, 5, 6, 7, 8, 11, 12, 15, 16, 17, 500)] == [0, 1, 3, 4, 4, 5, 5, 6, 6, 7, 7, 7, 7, 7]
    for rows, reach, window in ((8, 16.0, None), (5, 9.0, 30), (12, 100.0, 7), (4, 3.5, None), (32, 240.0, 200)):
        part = GroupedQueryAttention(BuildContext(torch.device("cpu"), torch.float32), "m", hidden_size=8, num_heads=2, num_kv_heads=1,
                                     head_dim=4, position=PartSpec("none"), window=window, bias=True, qk_norm_eps=1e-6,
                                     distance_bias={"rows": rows, "reach": reach}, force_general=True)
        table = torch.arange(rows * 2, dtype=torch.float32).view(rows, 2)
        laid = part._bias_by_distance(table)
        span = laid.shape[1]
        assert span >= (min(window, math.ceil(reach) + 1) if window else math.ceil(reach) + 1)
        for n in range(600):
            if window is not None and n >= window:
                break
            want = table[plain.distance_bucket(n, rows, reach)]
            assert torch.equal(laid[:, min(n, span - 1)], want), (rows, reach, n)


def test_attention_reference_at_the_window_s_edges():
    """The kernels' reference against the plain function with one key made to stand out: just inside and
    just outside the window, at a page's border, at the first position, for portions and single tokens."""
    g = torch.Generator().manual_seed(3)
    heads, groups, dim, vdim, block = 4, 2, 8, 6, 4
    for window, length, q_len in ((5, 23, 1), (5, 23, 6), (8, 16, 16), (12, 9, 1), (4, 17, 2), (1, 7, 3)):
        for edge in ("inside", "outside", "first"):
            sizes = {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": vdim, "scale": 0.7, "mask": {"size": window}, "bias_max": 9.0}
            w = {"m.q": torch.randn(heads * dim, 10, generator=g, dtype=F64), "m.k": torch.randn(groups * dim, 10, generator=g, dtype=F64),
                 "m.v": torch.randn(groups * vdim, 10, generator=g, dtype=F64), "m.q.b": torch.zeros(heads * dim, dtype=F64),
                 "m.k.b": torch.zeros(groups * dim, dtype=F64), "m.v.b": torch.zeros(groups * vdim, dtype=F64),
                 "m.q.norm": torch.ones(dim, dtype=F64), "m.k.norm": torch.ones(dim, dtype=F64),
                 "m.rel": torch.randn(6, heads, generator=g, dtype=F64), "m.o": torch.eye(heads * vdim, dtype=F64),
                 "m.o.b": torch.zeros(heads * vdim, dtype=F64)}
            h = torch.randn(length, 10, generator=g, dtype=F64)
            last = length - 1
            target = {"inside": max(last - window + 1, 0), "outside": max(last - window, 0), "first": 0}[edge]
            h[target] = 5.0 * h[last]           # a key that points where the last query points
            positions = torch.arange(length)
            want = plain.windowed_attention(h, w, "m", sizes, 1e-6, positions)
            q = plain.rms_norm((h @ w["m.q"].T).view(length, heads, dim), w["m.q.norm"], 1e-6)
            k = plain.rms_norm((h @ w["m.k"].T).view(length, groups, dim), w["m.k.norm"], 1e-6)
            v = (h @ w["m.v"].T).view(length, groups, vdim)
            pages = -(-length // block)
            perm = torch.randperm(pages + 2, generator=g)[:pages]
            key_pages = torch.full((pages + 2, groups, block, dim), float("nan"))
            value_pages = torch.full((pages + 2, groups, vdim, block), float("nan"))
            for p in range(length):
                key_pages[perm[p // block], :, p % block] = k[p].float()
                value_pages[perm[p // block], :, :, p % block] = v[p].float()
            laid = torch.stack([w["m.rel"][plain.distance_bucket(n, 6, 9.0)] for n in range(window)], dim=1).float()
            out = torch.zeros(q_len, heads * vdim)
            kernel_refs.masked_attention(q[length - q_len:].reshape(q_len, -1).float(), key_pages, value_pages, out,
                                         torch.tensor([0, q_len]), torch.tensor([length]), perm.view(1, -1).to(torch.int32), num_seqs=1,
                                         max_q_len=q_len, q_heads=heads, kv_heads=groups, head_dim=dim, value_dim=vdim, scale=0.7,
                                         window=window, dist_bias=laid)
            assert torch.allclose(out.double(), want[length - q_len:], atol=2e-4), (window, length, q_len, edge)


def test_expert_choice_reference_against_the_plain_choice():
    """Scores of all experts, corrections that can be negative, groups of which some are kept: the reference
    of the selection kernel chooses what the plain function chooses, and weighs it alike."""
    g = torch.Generator().manual_seed(11)
    for experts, top, groups, keep in ((12, 3, 4, 2), (6, 2, 1, 1), (8, 8, 2, 2), (9, 1, 3, 1), (16, 4, 2, 1), (5, 5, 5, 5)):
        x = torch.randn(40, 12, generator=g)
        router = torch.randn(experts + 1, 12, generator=g)
        correction = torch.randn(experts, generator=g) * 0.3 - 0.2
        chosen, weights, logits = kernel_refs.moe_route_grouped(x, router, correction, experts=experts, top=top, groups=groups,
                                                                 keep=keep, scale=2.25)
        assert logits.shape == (40, experts + 1)
        scores = torch.softmax((x.double() @ router[:experts].double().T), dim=-1)
        for t in range(40):
            want, _ = plain.choose_experts(scores[t], correction.double(), top, groups, keep)
            assert chosen[t].tolist() == want, (experts, t)
            total = sum(float(scores[t, e]) for e in want)
            assert torch.allclose(weights[t].double(), torch.tensor([float(scores[t, e]) / total * 2.25 for e in want], dtype=F64), atol=1e-5)


def test_norm_and_activation_references():
    g = torch.Generator().manual_seed(2)
    h, u, w = torch.randn(7, 20, generator=g), torch.randn(3, 7, 20, generator=g) * 4.0 + 1.5, torch.randn(20, generator=g)
    want = h.double() + 0.7 * plain.layer_norm(u.double().sum(0), w.double(), 1e-5)
    out = torch.zeros(7, 20)
    kernel_refs.layernorm_update(h, u, w, 1e-5, 0.7, out)
    assert torch.allclose(h.double(), want, atol=1e-5) and torch.equal(out, h)
    z = torch.randn(50, generator=g) * 3.0
    assert torch.allclose(kernel_refs.activate(z, "gelu").double(), plain.gelu_erf(z.double()), atol=1e-6)
