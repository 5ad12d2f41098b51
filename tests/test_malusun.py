"""Malusun through the engine on the CPU, with the kernels' plain references patched in, against the
plain implementation (tests/plain_malusun.py): configuration and tensor names, each mechanism alone,
and that logits do not depend on how requests are cut into steps, batched, or placed in pages and
state slots.  The kernels themselves run in the GPU tests."""

from __future__ import annotations

import copy
from types import SimpleNamespace

import pytest
import torch

import kernel_refs
import malusun_util as mu
import replay_util as ru
from forge_engine_amd.config import ConfigError, SchedulerConfig, load_model_config
from forge_engine_amd.engine import build_engine, load_model
from forge_engine_amd.sampling import SamplingParams
from forge_engine_amd.weights.random_init import declared_tensors

plain = mu.plain
LENGTHS = {"A": (5, 1, 14, 31), "B": (2, 9, 47, 23), "C": (7, 18, 3, 1), "D": (12, 1, 25, 6)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: mu.write_model(raw, 7, tmp_path_factory.mktemp(f"malusun_{name}")) for name, raw in mu.CONFIGS.items()}


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": mu.CONFIGS[name]["vocab"]}, seed, lengths)


def test_configuration_names_and_shapes():
    config = load_model_config(mu.SMALL_A)
    assert config.architecture == "Malusun" and load_model_config(config.to_dict()) == config
    tensors = declared_tensors(config)
    for name, shape in {"embed": (96, 48), "head": (96, 48), "final.norm": (48,), "l0.norm1": (48,), "l0.norm2b": (48,),
                        "l0.mix.in": (80, 48), "l0.mix.conv": (40, 4), "l0.mix.conv.b": (40,), "l0.mix.x": (17, 40),
                        "l0.mix.dt": (40, 5), "l0.mix.dt.b": (40,), "l0.mix.A_log": (40, 6), "l0.mix.D": (40,),
                        "l0.mix.o": (48, 40), "l0.mlp.up": (56, 48), "l0.mlp.down": (48, 56), "l1.mix.q": (64, 48),
                        "l1.mix.k": (32, 48), "l1.mix.v": (24, 48), "l1.mix.vmix": (), "l1.mix.o": (48, 48),
                        "l1.mlp.router": (5, 48), "l1.mlp.e4.gate": (20, 48), "l1.mlp.e0.down": (48, 20),
                        "l1.mlp.shared.up": (28, 48), "l2.mix.q.b": (48,), "l2.mix.k.b": (16,), "l2.mix.v.b": (24,),
                        "l2.mix.vmix": (), "l2.mlp.e2.up": (12, 48), "l3.mix.o": (48, 24), "l3.norm1b": (48,)}.items():
        assert tuple(tensors[name].shape) == shape, name
    # rotary attention has no biases, a router none, a layer without a feed-forward no norms around one
    assert not any(n in tensors for n in ("l1.mix.q.b", "l1.mlp.router.b", "l2.mlp.shared.up", "l3.norm2", "l3.norm2b", "l2.mix.o.b"))
    assert not any(n.startswith("l3.mlp") for n in tensors)
    unmixed = declared_tensors(load_model_config(mu.SMALL_D))
    assert "l0.mix.vmix" not in unmixed and "l1.mix.vmix" not in unmixed
    a = mu.SMALL_A
    for broken in ({**a, "layers": []},
                   {**a, "layers": [{**a["layers"][0], "type": "mamba3"}]},
                   {**a, "layers": [mu.layer(mu.attention(3, 2, 8, 8, 4, 4), None)]},           # heads no multiple of kv heads
                   {**a, "layers": [mu.layer(mu.attention(2, 2, 8, 8, 4, 10), None)]},          # more rotated dims than dims
                   {**a, "layers": [mu.layer(mu.attention(2, 2, 8, 8, 0, 4), None)]},           # an empty window
                   {**a, "layers": [mu.layer(mu.scan(16, 300, 2, 2), None)]},
                   {**a, "layers": [mu.layer(mu.scan(16, 4, 2, 9), None)]},
                   {**a, "layers": [mu.layer(mu.attention_2(2, 2, 8, 8, 4), mu.moe(2, 3, 8))]},   # more chosen than there are
                   {**a, "layers": [mu.layer(mu.attention_2(2, 2, 8, 8, 4), {"kind": "glu", "ff": 8})]},
                   {**a, "layers": [a["layers"][1], mu.layer(mu.attention_2(2, 2, 8, 16, 4), None)]},   # mixed values of two widths
                   {k: v for k, v in a.items() if k != "norm"}):
        with pytest.raises(ConfigError):
            load_model_config(broken)


def test_plain_in_steps_equals_plain_whole(folders):
    """The plain implementation's own pin: a request run from explicit state, token by token and in
    portions, gives the logits of the whole-sequence functions."""
    for name in ("A", "B", "C"):
        cfg, weights = mu.folder_weights(folders[name])
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
    got = ru.run_trace(folders[name], "float32", trace, tmp_path, block_size=mu.BLOCK_SIZE[name], device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders[name], requests), "float32")


def test_decoding_from_the_first_token_and_far_past_every_window(folders, tmp_path, monkeypatch):
    """One token a step from position 0 on, 75 steps: every window (5, 9, 13) passes over decoded tokens
    many times and pages go back to the pool while the request lives."""
    kernel_refs.install(monkeypatch)
    requests = requests_of("A", 8, (75,))
    trace = ru.trace_tail(requests, 75)
    assert len(trace.steps) == 75
    got = ru.run_trace(folders["A"], "float32", trace, tmp_path, block_size=4, device="cpu", on_cpu=True)
    mu.compare(got, mu.plain_logits(folders["A"], requests), "float32")


def test_pages_and_state_slots_are_used_again(folders, tmp_path, monkeypatch):
    """Seven requests through four state slots and a pool smaller than their sum: a request's recurrence
    and convolution start from nothing, whoever held the slot before."""
    kernel_refs.install(monkeypatch)
    for name in ("A", "C"):
        requests = requests_of(name, 4, (12, 20, 7, 16, 9, 3, 11))
        trace = ru.trace_mixed(requests, 9, max_live=4)
        assert sum(ru.round64(len(t)) for t in requests.values()) > trace.peak_tokens
        got = ru.run_trace(folders[name], "float32", trace, tmp_path / name, block_size=mu.BLOCK_SIZE[name], device="cpu", on_cpu=True)
        mu.compare(got, mu.plain_logits(folders[name], requests), "float32")


def test_greedy_generation_through_the_scheduler(folders, monkeypatch):
    kernel_refs.install(monkeypatch)
    _, model = load_model(folders["A"], dtype="float32", device="cpu")
    engine = build_engine(model, scheduler_config=SchedulerConfig(block_size=4, block_capacity=64, token_budget=8, max_batch_size=3),
                          eos_token_ids=())
    prompts = list(requests_of("A", 6, (11, 4, 17)).values())
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=6)) for prompt in prompts]
    engine.run_until_idle()
    cfg, weights = mu.folder_weights(folders["A"])
    for request_id, prompt in zip(ids, prompts):
        tokens = list(prompt)
        for _ in range(6):
            tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
        assert list(engine.request(request_id).output_token_ids) == tokens[len(prompt):]


# ------------------------------------------------------------------ windows and far keys, made to show

SHARP = mu.config(80, 32, [
    mu.layer(mu.attention(2, 1, 8, 8, 6, 4, base=50.0, scale=1.0), None),
    mu.layer(mu.attention_2(2, 1, 8, 8, 11, scale=1.0), None),
    mu.layer(mu.scan(24, 4, 3, 3), None),
])


def sharpen(tensors):
    """Queries and keys ten times as large: the softmax of every head sits on a few keys, so one key that
    is wrongly seen, or wrongly left out, moves the result; decays near one, so the recurrence remembers
    hundreds of tokens."""
    for name in tensors:
        if name.endswith((".mix.q", ".mix.k")):
            tensors[name] = (tensors[name].float() * 10.0).to(tensors[name].dtype)
        if name.endswith(".A_log"):
            tensors[name] = torch.full_like(tensors[name], -5.0)
        if name.endswith(".dt.b"):
            tensors[name] = torch.full_like(tensors[name], -3.0)


def test_a_window_one_token_off_or_a_lost_state_would_show(tmp_path, monkeypatch):
    """Sharp attention and a long memory, in portions and single tokens, against the plain implementation;
    and the control: the plain implementation itself with a window one token longer or shorter, without
    the one in the denominator, or without the first token, lands far outside the bound."""
    kernel_refs.install(monkeypatch)
    folder = mu.write_model(SHARP, 21, tmp_path / "model", change=sharpen)
    requests = requests_of("A", 12, (61, 38))
    requests = {k: [t % 80 for t in v] for k, v in requests.items()}
    want = mu.plain_logits(folder, requests)
    for mode, trace in (("portions", ru.trace_portions(requests)), ("tail", ru.trace_tail(requests, 30)),
                        ("mixed", ru.trace_mixed(requests, 3, max_live=2))):
        got = ru.run_trace(folder, "float32", trace, tmp_path / mode, block_size=4, device="cpu", on_cpu=True)
        mu.compare(got, want, "float32")
    cfg, weights = mu.folder_weights(folder)
    tokens = requests["r0"]
    right = plain.forward(cfg, weights, tokens)[-1]
    bound = 1e-5 + 1e-4 * float(right.abs().max())
    for layer, delta in ((0, 1), (0, -1), (1, 1), (1, -1)):
        other = copy.deepcopy(cfg)
        other["layers"][layer]["mixer"]["mask"]["size"] += delta
        assert float((plain.forward(other, weights, tokens)[-1] - right).abs().max()) > 100 * bound, (layer, delta)
    other = copy.deepcopy(cfg)
    other["layers"][1]["type"] = "attention"           # no one in the denominator, no slopes (and a rotation of nothing)
    other["layers"][1]["mixer"]["rot"] = {"dims": 2, "base": 1e30}
    assert float((plain.forward(other, weights, tokens)[-1] - right).abs().max()) > 100 * bound
    changed = [(tokens[0] + 1) % 80] + tokens[1:]       # the recurrence carries the first token to the last
    assert float((plain.forward(cfg, weights, changed)[-1] - right).abs().max()) > 5 * bound


def test_attention_reference_at_the_window_s_edges():
    """The kernels' reference against the plain function with one key made to stand out: just inside and
    just outside the window, at a page's border, at the first position, for portions and single tokens."""
    g = torch.Generator().manual_seed(3)
    heads, groups, dim, vdim, block = 4, 2, 8, 6, 4
    for window, length, q_len in ((5, 23, 1), (5, 23, 6), (8, 16, 16), (12, 9, 1), (4, 17, 2), (1, 7, 3)):
        for edge in ("inside", "outside", "first"):
            q = torch.randn(length, heads, dim, generator=g, dtype=torch.float64)
            k = torch.randn(length, groups, dim, generator=g, dtype=torch.float64)
            v = torch.randn(length, groups, vdim, generator=g, dtype=torch.float64)
            last = length - 1
            target = {"inside": max(last - window + 1, 0), "outside": max(last - window, 0), "first": 0}[edge]
            k[target] = 6.0 * q[last, ::heads // groups] / q[last, ::heads // groups].norm(dim=-1, keepdim=True)   # the last query's favourite
            positions = torch.arange(length)
            for slopes, one_more in ((None, False), (plain.distance_slopes(heads), True)):
                want = plain.windowed_attention(q, k, v, positions, positions, scale=1.0, window=window, slopes=slopes, one_more=one_more)
                pages = (length + block - 1) // block
                key_pages = torch.zeros(pages + 1, groups, block, dim)
                value_pages = torch.zeros(pages + 1, groups, vdim, block)
                table = torch.arange(pages, 0, -1, dtype=torch.int32).view(1, pages)     # pages in falling order, page 0 unused
                for p in range(length):
                    key_pages[int(table[0, p // block]), :, p % block] = k[p].float()
                    value_pages[int(table[0, p // block]), :, :, p % block] = v[p].float()
                out = torch.zeros(q_len, heads * vdim)
                kernel_refs.masked_attention(
                    q[length - q_len:].reshape(q_len, heads * dim).float(), key_pages, value_pages, out,
                    torch.tensor([0, q_len], dtype=torch.int32), torch.tensor([length], dtype=torch.int32), table, num_seqs=1,
                    max_q_len=q_len, q_heads=heads, kv_heads=groups, head_dim=dim, value_dim=vdim, scale=1.0, window=window,
                    sink=torch.zeros(heads) if one_more else None, slopes=None if slopes is None else slopes.float())
                assert torch.allclose(out.double(), want[length - q_len:].reshape(q_len, heads * vdim), atol=2e-5), (window, length, q_len, edge)


# ------------------------------------------------------------------ each mechanism alone

def _ctx():
    from forge_engine_amd.parts.base import BuildContext
    return BuildContext(torch.device("cpu"), torch.float32)


def _batch(q_lens, before, slots):
    """The metadata of a step: sequence i brings q_lens[i] tokens behind before[i] cached ones."""
    positions, token_seq, cu_q = [], [], [0]
    for i, (n, b) in enumerate(zip(q_lens, before)):
        positions += list(range(b, b + n))
        token_seq += [i] * n
        cu_q.append(cu_q[-1] + n)
    return SimpleNamespace(num_tokens=cu_q[-1], num_seqs=len(q_lens), positions=torch.tensor(positions, dtype=torch.int32),
                           token_seq=torch.tensor(token_seq, dtype=torch.int32), cu_q=torch.tensor(cu_q, dtype=torch.int32),
                           state_slots=torch.tensor(slots, dtype=torch.int32), carry={})


def _fill(part, generator, scale=0.3):
    weights = {}
    for name, spec in part.param_specs().items():
        weights[name] = torch.randn(spec.shape, generator=generator) * scale
        part.set_param(name, weights[name].clone())
    part.finalize()
    return {name: t.double() for name, t in weights.items()}


@pytest.mark.parametrize("sizes", [dict(inner=12, state=5, dt_rank=3, conv=4), dict(inner=8, state=17, dt_rank=1, conv=1),
                                   dict(inner=20, state=1, dt_rank=6, conv=2)])
def test_selective_scan_across_steps(sizes, monkeypatch):
    """Two sequences fed in pieces of unequal size through one part, their slots dirty from an earlier
    request and cleared at their start: the state and the convolution's last rows carry over."""
    from forge_engine_amd.cache.spec import CacheView
    from forge_engine_amd.parts.selective_scan import SelectiveScanMixer
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(sizes["inner"])
    width = 10
    part = SelectiveScanMixer(_ctx(), "m", hidden_size=width, inner=sizes["inner"], state=sizes["state"],
                              dt_rank=sizes["dt_rank"], conv_taps=sizes["conv"])
    w = _fill(part, g)
    inputs = [torch.randn(11, width, generator=g), torch.randn(6, width, generator=g)]
    want = [plain.selective_scan_mixer(x.double(), w, "m", sizes) for x in inputs]
    states = {name: torch.full((4, *spec.shape), 3.0) for name, spec in part.cache_needs().states().items()}
    for tensor in states.values():
        tensor[[2, 0]] = 0.0
    for step in ([(0, 5), (0, 1)], [(5, 6), (1, 4)], [(6, 11), (4, 6)]):
        batch = _batch([b - a for a, b in step], [a for a, _ in step], [2, 0])
        x = torch.cat([rows[a:b] for (a, b), rows in zip(step, inputs)])
        got = part.forward(x, batch, CacheView(states=states))
        at = 0
        for (a, b), expected in zip(step, want):
            assert torch.allclose(got[at:at + b - a].double(), expected[a:b], atol=1e-5), (sizes, step)
            at += b - a
    assert float(states[part.STATE][1].min()) == 3.0         # nobody else's slot was touched


@pytest.mark.parametrize("experts,top,shared", [(5, 2, 12), (3, 3, None), (4, 1, 6), (1, 1, None)])
def test_expert_mixture_alone(experts, top, shared, monkeypatch):
    from forge_engine_amd.models.malusun import EXPERT_NAMES
    from forge_engine_amd.parts.moe import RoutedExperts
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(experts * 10 + top)
    width, ff = 14, 9
    part = RoutedExperts(_ctx(), "f", hidden_size=width, experts=experts, top=top, intermediate_size=ff, shared_size=shared,
                         scoring="sigmoid", form="silu", weight_input=True, router_bias=False, names=EXPERT_NAMES)
    w = _fill(part, g, 0.5)
    x = torch.randn(13, width, generator=g)
    mlp = mu.moe(experts, top, ff, shared)
    want = plain.expert_mixture(x.double(), w, "f", mlp)
    got = part.forward(x, None)
    assert got.shape == (top, 13, width)          # one part a choice, added up in order by whoever reads them
    assert torch.allclose(got.sum(0).double(), want, atol=1e-5)
    # the weight is on the input: doubling every score's expert input is not doubling its output
    one = plain.gated_expert(x.double(), w, "f.e0")
    assert not torch.allclose(plain.gated_expert(0.5 * x.double(), w, "f.e0"), 0.5 * one, atol=1e-3)


def test_dense_feed_forward_norms_and_embedding(monkeypatch):
    from forge_engine_amd.parts.base import Residual
    from forge_engine_amd.parts.block import SandwichNormBlock
    from forge_engine_amd.parts.embedding import TokenEmbedding
    from forge_engine_amd.parts.mlp import ActivatedMLP
    from forge_engine_amd.parts.norm import RMSNorm
    kernel_refs.install(monkeypatch)
    g = torch.Generator().manual_seed(2)
    width, tokens, eps = 10, 7, 1e-3
    feed = ActivatedMLP(_ctx(), "f", hidden_size=width, intermediate_size=16)
    w = _fill(feed, g, 0.5)
    x = torch.randn(tokens, width, generator=g)
    assert torch.allclose(feed.forward(x, None).double(), plain.dense_feed_forward(x.double(), w, "f"), atol=1e-5)

    embedding = TokenEmbedding(_ctx(), "embed", vocab_size=30, hidden_size=width, leaf="", scale=0.3)
    table = _fill(embedding, g, 1.0)["embed"]
    ids = torch.tensor([3, 29, 0, 3], dtype=torch.int32)
    assert torch.allclose(embedding.forward(SimpleNamespace(num_tokens=4, token_ids=ids)).h.double(), table[ids.long()] * 0.3, atol=1e-6)

    # a layer around plain functions as sublayers; the mixer's update comes in two parts
    a, b = torch.randn(width, width, generator=g), torch.randn(width, width, generator=g)

    class Mixer:
        def forward(self, h, batch, cache, writes_cache=True):
            y = torch.tanh(h.float() @ a)
            return torch.stack([0.25 * y, 0.75 * y])

        def cache_needs(self):
            return None

    class FeedForward:
        def forward(self, h, batch):
            return torch.sin(h.float() @ b)

    norms, nw = {}, {}
    for role in SandwichNormBlock.NORMS + ("last",):
        norms[role] = RMSNorm(_ctx(), role, size=width, eps=eps, leaf="", offset=1.0)
        nw[role] = _fill(norms[role], g, 0.2)[role]
    for with_feed_forward in (True, False):
        block = SandwichNormBlock(_ctx(), Mixer(), FeedForward() if with_feed_forward else None, norms)
        x0 = torch.randn(tokens, width, generator=g)
        residual = Residual(x0.clone())
        block.forward(residual, None, None)
        block.forward(residual, None, None)          # a second layer: the norm behind meets the next norm before
        rows = torch.tensor([5, 0], dtype=torch.int32)
        got = norms["last"].forward(residual, rows=rows)
        h = x0.double()
        for _ in range(2):
            h = h + plain.offset_norm(torch.tanh(plain.offset_norm(h, nw["input"], eps) @ a.double()), nw["mixer_out"], eps)
            if with_feed_forward:
                h = h + plain.offset_norm(torch.sin(plain.offset_norm(h, nw["post_mixer"], eps) @ b.double()), nw["ff_out"], eps)
        assert torch.allclose(got.double(), plain.offset_norm(h, nw["last"], eps)[rows.long()], atol=1e-5)
        assert torch.allclose(residual.flush().double(), h, atol=1e-5)
