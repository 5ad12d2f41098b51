"""Malusun on the GPU: its kernels alone against their plain references (tests/kernel_refs.py), and
the model against the plain implementation (tests/plain_malusun.py) in float32 and bfloat16 over
traces that cut the same requests in different ways."""

from __future__ import annotations

import pytest
import torch

import kernel_refs as refs
import malusun_util as mu
import replay_util as ru

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
plain = mu.plain

CONFIGS = dict(mu.CONFIGS, M=mu.MEDIUM)
LENGTHS = {"A": (5, 1, 14, 27, 90), "B": (2, 9, 21, 33, 64), "C": (7, 18, 3, 1, 40), "D": (12, 1, 25, 6, 50), "M": (4, 45, 150, 83, 1)}
BLOCKS = dict(mu.BLOCK_SIZE, M=16)


def close(got, want, dtype, loose=1.0):
    if dtype == torch.float32:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-5 * loose, atol=2e-5 * loose)
    else:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-2 * loose, atol=2e-2 * loose)


def to_dev(*tensors):
    return [None if t is None else t.to(DEV) for t in tensors]


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("channels,states,taps", [(40, 6, 4), (24, 16, 1), (300, 3, 2), (64, 22, 3), (130, 40, 8), (16, 100, 4), (8, 200, 2),
                                                  (2048, 16, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolution_and_selective_scan_kernels(channels, states, taps, dtype):
    """Sequences of unequal length in one step (one of a single token, one longer than a chunk, an empty
    one that pads the step with a slot beyond the pool), twice in a row so that the second step starts from
    the state the first left; inputs read through strided views; every shape of the scan (lanes a channel
    times states a lane) comes up over the sizes."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(channels + states)
    slots = 5
    weight, bias = torch.randn(channels, taps, generator=g) * 0.4, torch.randn(channels, generator=g) * 0.1
    a = -torch.exp(torch.randn(channels, states, generator=g) * 0.5)
    d, dt_bias = torch.randn(channels, generator=g), torch.randn(channels, generator=g) * 0.5 - 1.0
    conv_ref, scan_ref = torch.randn(slots, max(taps - 1, 1), channels, generator=g), torch.randn(slots, channels, states, generator=g)
    conv_gpu, scan_gpu = conv_ref.clone().to(DEV), scan_ref.clone().to(DEV)
    for q_lens in ([1, 37, 0, 5], [3, 1, 0, 16]):
        tokens = sum(q_lens)
        cu = [0]
        for n in q_lens:
            cu.append(cu[-1] + n)
        cu_q = torch.tensor(cu, dtype=torch.int32)
        token_seq = torch.tensor([s for s, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32)
        state_slots = torch.tensor([3, 0, slots, 4], dtype=torch.int32)        # the empty sequence's slot is beyond the pool
        xz = torch.randn(tokens, 2 * channels + 3, generator=g).to(dtype)
        bc = torch.randn(tokens, 2 * states + 5, generator=g)
        dt_lin = torch.randn(tokens, channels, generator=g)
        want_u = refs.causal_conv_act(xz[:, :channels], weight, bias, conv_ref if taps > 1 else None, token_seq, cu_q, state_slots,
                                      num_seqs=4, act="silu")
        got_u = ops.causal_conv_act(xz.to(DEV)[:, :channels], weight.to(DEV), bias.to(DEV), conv_gpu if taps > 1 else None,
                                    token_seq.to(DEV), cu_q.to(DEV), state_slots.to(DEV), num_seqs=4, act="silu")
        close(got_u, want_u, dtype)
        if taps > 1:
            close(conv_gpu, conv_ref, torch.float32)
        z = xz[:, channels + 3:]
        want = refs.selective_scan(want_u, dt_lin, dt_bias, a, bc[:, 5:], d, z, scan_ref, cu_q, state_slots, num_seqs=4)
        got = ops.selective_scan(want_u.to(DEV), dt_lin.to(DEV), dt_bias.to(DEV), a.to(DEV), bc.to(DEV)[:, 5:], d.to(DEV),
                                 xz.to(DEV)[:, channels + 3:], scan_gpu, cu_q.to(DEV), state_slots.to(DEV), num_seqs=4)
        close(got, want, dtype, loose=5.0)
        close(scan_gpu, scan_ref, torch.float32, loose=5.0)


@pytest.mark.parametrize("segment,q_lens", [(16, [70, 1, 0, 33]), (32, [200, 31, 0, 97]), (128, [700, 3, 0, 129]), (64, [64, 128, 0, 65])])
@pytest.mark.parametrize("channels,states", [(40, 6), (96, 16), (24, 40)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_selective_scan_in_segments(monkeypatch, segment, q_lens, channels, states, dtype):
    """A step whose sequences are cut into segments that are walked side by side: lengths that end on a
    segment's edge, one token behind it and one short of it, a sequence inside one segment, an empty one;
    twice in a row, so that the second step starts from the state the segments' last walk left.  Decays near
    one, so that a segment's start state matters to its end."""
    from forge_engine_amd.kernels import ops
    monkeypatch.setattr(ops, "SCAN_SEGMENT", segment)
    monkeypatch.setattr(ops, "SCAN_SEGMENT_MIN_TOKENS", 1)
    g = torch.Generator().manual_seed(channels + states + segment)
    slots = 5
    a = -torch.exp(torch.randn(channels, states, generator=g) * 0.5 - 2.0)
    d, dt_bias = torch.randn(channels, generator=g), torch.randn(channels, generator=g) * 0.5 - 2.0
    scan_ref = torch.randn(slots, channels, states, generator=g)
    scan_gpu = scan_ref.clone().to(DEV)
    for lens in (q_lens, q_lens[::-1]):
        tokens = sum(lens)
        assert ops.scan_segment(tokens, 4) == segment
        cu_q = torch.tensor([sum(lens[:i]) for i in range(5)], dtype=torch.int32)
        state_slots = torch.tensor([3, 0, 1, 4] if lens is q_lens else [4, slots, 0, 3], dtype=torch.int32)
        if lens is not q_lens:       # the empty sequence is the second one now
            assert lens[1] == 0
        else:
            state_slots[2] = slots
        x = torch.randn(tokens, channels, generator=g).to(dtype)
        z = torch.randn(tokens, channels, generator=g).to(dtype)
        bc = torch.randn(tokens, 2 * states, generator=g)
        dt_lin = torch.randn(tokens, channels, generator=g)
        want = refs.selective_scan(x, dt_lin, dt_bias, a, bc, d, z, scan_ref, cu_q, state_slots, num_seqs=4)
        got = ops.selective_scan(*to_dev(x, dt_lin, dt_bias, a, bc, d, z), scan_gpu, cu_q.to(DEV), state_slots.to(DEV), num_seqs=4)
        close(got, want, dtype, loose=5.0)
        close(scan_gpu, scan_ref, torch.float32, loose=5.0)


@pytest.mark.parametrize("taps,q_lens", [(4, [530, 1, 0, 501]), (2, [17, 1000, 0, 15]), (8, [3, 2, 0, 1040]), (1, [600, 400, 0, 48])])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolution_over_runs_of_rows(taps, q_lens, dtype):
    """A step large enough for the convolution's wide shape (four channels a thread, rows in runs that keep
    the taps' rows in registers): sequences that begin inside a run, at its first and at its last row, so
    that rows of the state and of another sequence's part of the step lie side by side; twice in a row."""
    from forge_engine_amd.kernels import ops
    channels, slots = 1024, 5
    g = torch.Generator().manual_seed(taps)
    weight, bias = torch.randn(channels, taps, generator=g) * 0.4, torch.randn(channels, generator=g) * 0.1
    conv_ref = torch.randn(slots, max(taps - 1, 1), channels, generator=g)
    conv_gpu = conv_ref.clone().to(DEV)
    for lens in (q_lens, q_lens[::-1]):
        tokens = sum(lens)
        cu_q = torch.tensor([sum(lens[:i]) for i in range(5)], dtype=torch.int32)
        token_seq = torch.tensor([s for s, n in enumerate(lens) for _ in range(n)], dtype=torch.int32)
        state_slots = torch.tensor([3, 0, 1, 4], dtype=torch.int32)
        state_slots[lens.index(0)] = slots
        xz = torch.randn(tokens, 2 * channels, generator=g).to(dtype)
        want = refs.causal_conv_act(xz[:, channels:], weight, bias, conv_ref if taps > 1 else None, token_seq, cu_q, state_slots,
                                    num_seqs=4, act="silu")
        got = ops.causal_conv_act(xz.to(DEV)[:, channels:], weight.to(DEV), bias.to(DEV), conv_gpu if taps > 1 else None,
                                  token_seq.to(DEV), cu_q.to(DEV), state_slots.to(DEV), num_seqs=4, act="silu")
        close(got, want, dtype)
        if taps > 1:
            close(conv_gpu, conv_ref, torch.float32)


def test_scan_shapes_cover_every_size():
    from forge_engine_amd.kernels import ops
    for states in range(1, 257):
        for channels, seqs in ((64, 1), (8192, 64)):
            lanes, per_lane = ops.scan_shape(channels, states, seqs)
            assert lanes * per_lane >= states and (lanes, per_lane) in ops._SCAN_SHAPES


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 12, 8), (2, 1, 128, 128, 64), (3, 3, 10, 6, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_values_leaning_on_another_layer_s(heads, kv_heads, dim, vdim, rot, dtype):
    """The page-write kernel with a bias: a layer that keeps its values for others, and one whose values
    become a blend with those before they are stored."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(dim)
    tokens, block, pages = 7, 4, 9
    channels = (heads + kv_heads) * dim + kv_heads * vdim
    qkv = torch.randn(tokens, channels + 2, generator=g).to(dtype)
    bias = torch.randn(channels, generator=g) * 0.3
    inv_freq = torch.rand(max(rot // 2, 1), generator=g)[:rot // 2] if rot else None
    positions = torch.tensor([0, 1, 2, 3, 9, 10, 30], dtype=torch.int32)
    token_seq = torch.tensor([0, 0, 0, 0, 1, 1, 2], dtype=torch.int32)
    cu_q, slots = torch.tensor([0, 4, 6, 7], dtype=torch.int32), torch.tensor([0, 1, 2], dtype=torch.int32)
    table = torch.full((3, 8), -1, dtype=torch.int32)
    table[0, 0], table[1, 2], table[2, 7] = 5, 2, 8
    v_from = torch.randn(tokens, kv_heads * vdim, generator=g).to(dtype)
    common = dict(num_seqs=3, q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, rotary_dim=rot, unit_norm_eps=None, taps=0)
    for mixing in ({}, {"v_keep": True}, {"v_from": v_from, "v_mix": 0.37}):
        outs = []
        for module, move in ((refs, lambda t: t), (ops, lambda t: None if t is None else t.to(DEV))):
            k = torch.zeros(pages, kv_heads, block, dim, dtype=dtype)
            v = torch.zeros(pages, kv_heads, vdim, block, dtype=dtype)
            q = torch.empty(tokens, heads * dim, dtype=dtype)
            extra = dict(mixing)
            if "v_keep" in extra:
                extra["v_keep"] = move(torch.zeros(tokens, kv_heads * vdim, dtype=dtype))
            if "v_from" in extra:
                extra["v_from"] = move(v_from)
            k, v, q = move(k), move(v), move(q)
            module.conv_rope_norm_write(move(qkv), move(bias), None, None, move(inv_freq), move(positions), move(token_seq), move(cu_q),
                                        move(slots), move(table), k, v, q, **common, **extra)
            outs.append((q, k, v, extra.get("v_keep")))
        for want, got in zip(*outs):
            if want is not None:
                close(got, want, dtype)
        if "v_keep" in mixing:      # what is kept is what was stored
            kept, stored = outs[1][3], outs[1][2]
            assert torch.equal(kept[0].view(kv_heads, vdim).cpu(), stored[5, :, :, 0].cpu())


@pytest.mark.parametrize("tokens,hidden,experts,top,inner", [(1, 48, 5, 2, 20), (37, 64, 3, 1, 36), (150, 256, 6, 2, 96), (70, 40, 4, 4, 100),
                                                             (600, 128, 4, 2, 160), (9, 64, 1, 1, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_with_sigmoid_scores_on_their_inputs(tokens, hidden, experts, top, inner, dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(tokens + experts)
    x = torch.randn(tokens, hidden, generator=g).to(dtype)
    router = (torch.randn(experts, hidden, generator=g) * 0.3).to(dtype)
    gate_up = (torch.randn(experts, 2 * inner, hidden, generator=g) * 0.1).to(dtype)
    down = (torch.randn(experts, hidden, inner, generator=g) * 0.1).to(dtype)
    want_chosen, want_weights = refs.moe_route(x, router, None, top, scoring="sigmoid")
    chosen, weights = ops.moe_route(x.to(DEV), router.to(DEV), None, top, scoring="sigmoid")
    assert torch.equal(chosen.cpu(), want_chosen)
    torch.testing.assert_close(weights.cpu(), want_weights, rtol=1e-4, atol=1e-5)
    assert experts == 1 or float((want_weights.sum(-1) - 1).abs().max()) > 0.05       # nothing is renormalised
    extra = torch.randn(2, tokens, hidden, generator=g)
    for weight_input in (True, False):
        want = refs.moe_experts(x, want_chosen, want_weights, gate_up, down, torch.empty(top, tokens, hidden), extra=extra, form="silu",
                                weight_input=weight_input)
        got = ops.moe_experts(x.to(DEV), chosen, weights, gate_up.to(DEV), down.to(DEV), torch.empty(top, tokens, hidden, device=DEV),
                              extra=extra.to(DEV), form="silu", weight_input=weight_input)
        close(got, want, dtype, loose=2.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_relu_squared_kernel(dtype):
    from forge_engine_amd.kernels import ops
    x = torch.randn(37, 130, generator=torch.Generator().manual_seed(1)).to(dtype)
    close(ops.relu_squared(x.to(DEV)), refs.relu_squared(x), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [4, 16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 24, 16), (6, 3, 64, 64), (8, 1, 128, 128), (2, 2, 10, 6)])
@pytest.mark.parametrize("window", [1, 7, 64, 150])
def test_one_key_at_the_window_s_edge(dtype, block_size, heads, kv_heads, dim, vdim, window):
    """Keys whose scores dominate sit just inside and just outside the window of the last token, of the
    portion's first token and of tokens between, at page borders and at the first position: the attention
    kernels against the plain windowed attention, with and without the distance penalty and the one in the
    denominator, for a prompt's portion behind cached keys and for single tokens."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(dim + block_size + window)
    length, cached = 230, 201
    q = torch.randn(length, heads, dim, generator=g)
    k = torch.randn(length, kv_heads, dim, generator=g)
    v = torch.randn(length, kv_heads, vdim, generator=g)
    loud = {0, block_size - 1, block_size}
    for p in (length - 1, cached, cached + 13, 215):
        loud |= {max(p - window, 0), max(p - window + 1, 0)}
    for far in loud:
        k[far] *= 4.0
    q, k, v = (t.to(dtype) for t in (q, k, v))
    positions = torch.arange(length)
    pages = -(-length // block_size)
    perm = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    key_pages = torch.zeros(pages + 3, kv_heads, block_size, dim, dtype=dtype)
    value_pages = torch.zeros(pages + 3, kv_heads, vdim, block_size, dtype=dtype)
    for p in range(length):
        key_pages[perm[p // block_size], :, p % block_size] = k[p]
        value_pages[perm[p // block_size], :, :, p % block_size] = v[p]
    key_pages, value_pages = key_pages.to(DEV), value_pages.to(DEV)
    table = perm.view(1, -1).to(DEV)
    for penalised in (False, True):
        slopes = plain.distance_slopes(heads) if penalised else None
        want = plain.windowed_attention(q.double(), k.double(), v.double(), positions, positions, scale=0.4, window=window,
                                        slopes=slopes, one_more=penalised).reshape(length, heads * vdim).float()
        common = dict(q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, scale=0.4, window=window,
                      sink=torch.zeros(heads, device=DEV) if penalised else None,
                      slopes=slopes.float().to(DEV) if penalised else None)
        out = torch.empty(length - cached, heads * vdim, dtype=dtype, device=DEV)
        ops.masked_attention(q[cached:].reshape(length - cached, -1).to(DEV), key_pages, value_pages, out,
                             torch.tensor([0, length - cached], dtype=torch.int32, device=DEV),
                             torch.tensor([length], dtype=torch.int32, device=DEV), table, num_seqs=1, max_q_len=length - cached,
                             num_decode=0, max_ctx=length, **common)
        close(out, want[cached:], dtype)
        places = [0, block_size - 1, block_size, window - 1, window, min(window + 1, length - 1), cached, length - 1]
        n = len(places)
        out = torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
        ops.masked_attention(q[places].reshape(n, -1).to(DEV), key_pages, value_pages, out,
                             torch.arange(n + 1, dtype=torch.int32, device=DEV),
                             torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV), table.expand(n, -1).contiguous(),
                             num_seqs=n, max_q_len=1, num_decode=n, max_ctx=length, **common)
        close(out, want[places], dtype)


# ------------------------------------------------------------------ the model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: mu.write_model(raw, 31, tmp_path_factory.mktemp(f"malusun_{name}")) for name, raw in CONFIGS.items()}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def expected(name, folder, cache, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in cache:
        cache[key] = mu.plain_logits(folder, requests)
    return cache[key]


def requests_of(name, seed, lengths):
    return ru.make_requests({"vocab_size": CONFIGS[name]["vocab"]}, seed, lengths)


TRACES = {
    "whole": ru.trace_whole,
    "tail": lambda r: ru.trace_tail(r, 32),
    "portions": ru.trace_portions,
    "mixed": lambda r: ru.trace_mixed(r, 5, max_live=4),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_matches_plain(name, mode, dtype, folders, plain_cache, tmp_path):
    requests = requests_of(name, 3, LENGTHS[name])
    trace = TRACES[mode](requests)
    print(f"replay {name} {mode} {dtype}: {len(trace.steps)} steps", flush=True)
    got = ru.run_trace(folders[name], dtype, trace, tmp_path, block_size=BLOCKS[name])
    worst = mu.compare(got, expected(name, folders[name], plain_cache, requests), dtype)
    print(f"  worst difference {worst:.3e}", flush=True)


def sharpen(tensors):
    """Queries four times as large and decays near one: a key at a window's edge, and the first token of
    hundreds, reach the logits."""
    for name in tensors:
        if name.endswith(".mix.q"):
            tensors[name] = (tensors[name].float() * 4.0).to(tensors[name].dtype)
        if name.endswith(".A_log"):
            tensors[name] = torch.full_like(tensors[name], -4.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_with_sharp_attention_and_a_long_memory(dtype, tmp_path):
    """Prompts of several hundred tokens, longer than every window: whole, then the last 40 tokens one by
    one (across page borders and the windows' edges), then in portions, then three at once."""
    folder = mu.write_model(mu.MEDIUM, 32, tmp_path / "sharp", change=sharpen)
    requests = requests_of("M", 9, (500, 333, 129))
    want = mu.plain_logits(folder, requests)
    for mode, trace in (("whole", ru.trace_whole(requests)), ("tail", ru.trace_tail(requests, 40)),
                        ("portions", ru.trace_portions(requests, sizes=(64, 17, 2, 130, 3, 48, 16, 2, 33), want_all=False)),
                        ("mixed", ru.trace_mixed(requests, 11, max_live=3))):
        print(f"sharp {mode} {dtype}: {len(trace.steps)} steps", flush=True)
        got = ru.run_trace(folder, dtype, trace, tmp_path / mode, block_size=16)
        mu.compare(got, want, dtype, fraction=0.1, float32_factor=10.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_equal_eager_steps_and_long_decoding(dtype, folders):
    """A prompt and then 150 single tokens, two requests side by side: steps replayed from captured graphs
    against the same steps run eagerly (the recurrent state moves on once a step either way), and both
    against the plain implementation."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["M"], dtype=dtype, device=DEV)
    requests = requests_of("M", 21, (160, 171))
    want = mu.plain_logits(folders["M"], requests)
    results = {}
    for graphs in (True, False):
        runner = ModelRunner(model, block_size=16, block_capacity=40, num_state_slots=3, use_graphs=graphs, eager_sightings=1)
        got = {}
        for name in requests:
            runner.begin(name)
        at = {"r0": 10, "r1": 21}
        logits = runner.step([StepEntry(n, requests[n][:at[n]], [at[n] - 1]) for n in requests])
        for row, n in zip(logits, requests):
            got[(n, at[n] - 1)] = row.cpu().clone()
        for _ in range(150):
            logits = runner.step([StepEntry(n, [requests[n][at[n]]], [0]) for n in requests])
            for row, n in zip(logits, requests):
                got[(n, at[n])] = row.cpu().clone()
                at[n] += 1
        assert runner.graph_replays >= (140 if graphs else 0) and (graphs or runner.graph_replays == 0)
        results[graphs] = got
        mu.compare(got, want, dtype, fraction=0.1)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=0, atol=0 if dtype == "float32" else 1e-2)


def test_first_tokens_and_slot_reuse(folders):
    """A request that takes over the state slot of one that ended starts from an empty state and empty
    convolution rows, whatever the slot still holds; requests of one and two tokens."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["A"], dtype="float32", device=DEV)
    runner = ModelRunner(model, block_size=4, block_capacity=16, num_state_slots=1)
    cfg, weights = mu.folder_weights(folders["A"])
    for tokens in ([5, 90, 17, 3], [44], [7, 7], [90, 5, 17, 3, 3, 3, 8, 1, 2]):
        runner.begin("only")
        rows = []
        for token in tokens:
            rows.append(runner.step([StepEntry("only", [token], [0])])[0].cpu().clone())
        runner.end("only")
        want = plain.forward(cfg, weights, tokens)
        for got, row in zip(rows, want):
            assert float((got.double() - row).abs().max()) <= 1e-5 + 1e-4 * float(row.abs().max())


def test_generation_through_the_entry_point_and_the_command_line(folders):
    import os
    import subprocess
    import sys
    from conftest import ROOT
    from forge_engine_amd.config import SchedulerConfig
    from forge_engine_amd.engine import engine_from_folder
    from forge_engine_amd.sampling import SamplingParams

    cfg, weights = mu.folder_weights(folders["A"])

    def greedy(prompt, count):
        tokens = list(prompt)
        for _ in range(count):
            tokens.append(int(plain.forward(cfg, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    prompts = list(requests_of("A", 13, (11, 3, 25)).values())
    want = [greedy(prompt, 8) for prompt in prompts]
    engine = engine_from_folder(folders["A"], scheduler_config=SchedulerConfig(block_size=4, block_capacity=128, token_budget=16),
                                dtype="float32", eos_token_ids=[])
    ids = [engine.submit(prompt, sampling_params=SamplingParams(max_new_tokens=8)) for prompt in prompts]
    engine.run_until_idle()
    assert [list(engine.request(i).output_token_ids) for i in ids] == want
    command = [sys.executable, str(ROOT / "bin" / "forge-engine"), "generate", "--model", str(folders["A"]), "--dtype", "float32",
               "--max-new-tokens", "8", "--block-size", "4", "--prompt-ids", ",".join(map(str, prompts[0]))]
    done = subprocess.run(command, capture_output=True, text=True, timeout=300, env=dict(os.environ))
    assert done.returncode == 0, done.stderr[-2000:]
    assert ",".join(map(str, want[0])) in done.stdout.replace(" ", "")


@pytest.mark.parametrize("rows,width,parts", [(1, 40, 1), (37, 256, 3), (9, 2048, 1), (600, 4096, 2), (5, 8192, 1), (3, 9000, 2), (11, 50, 2), (530, 1022, 1), (2100, 2048, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_norms_in_one_kernel(rows, width, parts, dtype):
    """The norm behind a sublayer and the norm before the next: whole steps (the stream moves on) and chosen rows
    (it does not), updates whole and in parts, rows wider than the fused kernel takes."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + width)
    h = torch.randn(rows, width, generator=g) * 2
    update = torch.randn(rows, width, generator=g) if parts == 1 else torch.randn(parts, rows, width, generator=g)
    w, w_next = 1 + 0.2 * torch.randn(width, generator=g), 1 + 0.2 * torch.randn(width, generator=g)
    pick = torch.tensor([rows - 1, 0, rows - 1], dtype=torch.int32)
    for chosen in (pick, None):
        want_h, got_h = h.clone(), h.clone().to(DEV)
        n = rows if chosen is None else chosen.numel()
        want = refs.rmsnorm_update_norm(want_h, update, w, 1e-5, w_next, 1e-6, torch.empty(n, width, dtype=dtype), rows=chosen)
        got = ops.rmsnorm_update_norm(got_h, update.to(DEV), w.to(DEV), 1e-5, w_next.to(DEV), 1e-6,
                                      torch.empty(n, width, dtype=dtype, device=DEV), rows=None if chosen is None else chosen.to(DEV))
        close(got, want, dtype)
        close(got_h, want_h, torch.float32)
        assert chosen is None or torch.equal(got_h.cpu(), h)
