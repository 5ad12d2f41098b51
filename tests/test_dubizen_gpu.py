"""Dubizen on the GPU: its kernels alone against their plain references (tests/kernel_refs.py), and
the model against the plain implementation (tests/plain_dubizen.py) in float32 and bfloat16 over
traces that cut the same requests in different ways."""

from __future__ import annotations

import pytest
import torch

import dubizen_util as du
import kernel_refs as refs
import replay_util as ru

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
plain = du.plain

CONFIGS = dict(du.CONFIGS, M=du.MEDIUM)
LENGTHS = {"A": (5, 1, 14, 27, 90), "B": (2, 9, 21, 33, 64), "C": (7, 18, 3, 1, 40), "D": (12, 1, 25, 6, 50), "M": (4, 45, 150, 83, 1)}
BLOCKS = dict(du.BLOCK_SIZE, M=16)


def close(got, want, dtype, loose=1.0):
    if dtype == torch.float32:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-5 * loose, atol=2e-5 * loose)
    else:
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=2e-2 * loose, atol=2e-2 * loose)


def to_dev(*tensors):
    return [None if t is None else t.to(DEV) for t in tensors]


# ------------------------------------------------------------------ kernels alone

@pytest.mark.parametrize("rows,width,parts", [(1, 40, 1), (37, 256, 3), (9, 2048, 1), (600, 4096, 2), (3, 9000, 2), (11, 50, 2), (530, 1022, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_norm_of_an_update(rows, width, parts, dtype):
    """Updates far from zero mean, whole and in parts, rows held in registers and rows read again."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + width)
    h = torch.randn(rows, width, generator=g)
    update = torch.randn(*((parts,) if parts > 1 else ()), rows, width, generator=g) * 3.0 + 2.0
    weight = 1.0 + torch.randn(width, generator=g) * 0.1
    want_h, want_out = h.clone(), torch.zeros(rows, width, dtype=dtype)
    refs.layernorm_update(want_h, update, weight, 1e-5, 0.7, want_out)
    got_h, got_out = h.clone().to(DEV), torch.empty(rows, width, dtype=dtype, device=DEV)
    ops.layernorm_update(got_h, update.to(DEV), weight.to(DEV), 1e-5, 0.7, got_out)
    close(got_h, want_h, torch.float32, loose=5.0)
    close(got_out, want_out, dtype, loose=5.0)
    again = h.clone().to(DEV)
    assert ops.layernorm_update(again, update.to(DEV), weight.to(DEV), 1e-5, 0.7, None) is None
    close(again, want_h, torch.float32, loose=5.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activations_and_row_gates(dtype):
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(37, 300, generator=g) * 3.0).to(dtype)
    for kind in ("gelu", "gelu_tanh", "relu_squared"):
        close(ops.activate(x.to(DEV), kind), refs.activate(x, kind), dtype)
    for shape in ((23, 64), (3, 23, 64)):
        update, logits = torch.randn(*shape, generator=g), torch.randn(23, 5, generator=g) * 2.0
        want = refs.gate_rows(update.clone(), logits, 3)
        close(ops.gate_rows(update.to(DEV), logits.to(DEV), 3), want, torch.float32)


@pytest.mark.parametrize("tokens,hidden,experts,top,groups,keep", [(1, 48, 6, 2, 2, 1), (37, 64, 9, 3, 3, 2), (150, 256, 16, 4, 4, 2), (70, 40, 4, 4, 1, 1),
                                                                   (300, 128, 64, 8, 8, 3), (5, 32, 12, 1, 12, 5), (70, 64, 256, 8, 8, 4),
                                                                   (129, 48, 192, 6, 16, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_choice_of_experts_within_the_best_groups(tokens, hidden, experts, top, groups, keep, dtype):
    """Corrections of both signs; a router with one more row whose logits come back untouched; the choice and
    the weights against the reference on the kernel's own logits, so that roundings cannot turn a choice."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(tokens + experts)
    x = torch.randn(tokens, hidden, generator=g).to(dtype)
    router = (torch.randn(experts + 1, hidden, generator=g) * 0.3).to(dtype)
    correction = torch.randn(experts, generator=g) * 0.2 - 0.1
    chosen, weights, logits = ops.moe_route_grouped(x.to(DEV), router.to(DEV), correction.to(DEV), experts=experts, top=top, groups=groups,
                                                    keep=keep, scale=1.75)
    assert logits.shape == (tokens, experts + 1)
    close(logits, x.float() @ router.float().T, dtype, loose=2.0)
    eye = torch.eye(experts + 1)          # the reference on the kernel's logits: x = logits, router = identity
    want_chosen, want_weights, _ = refs.moe_route_grouped(logits.cpu(), eye, correction, experts=experts, top=top, groups=groups, keep=keep, scale=1.75)
    assert torch.equal(chosen.cpu(), want_chosen)
    close(weights, want_weights, torch.float32, loose=5.0)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 12, 0), (2, 1, 128, 128, 64), (3, 3, 10, 6, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_weighted_norms_of_q_and_k_heads_before_the_page_write(heads, kv_heads, dim, vdim, rot, dtype):
    """Biases, the weighted RMS norm of every q and k head (before the rotation where there is one), q out,
    k and v into their pages."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(dim)
    tokens, block, pages = 21, 4, 8
    channels = (heads + kv_heads) * dim + kv_heads * vdim
    qkv = torch.randn(tokens, channels + 3, generator=g).to(dtype)
    bias = torch.randn(channels, generator=g) * 0.3
    wq, wk = 1.0 + torch.randn(dim, generator=g) * 0.3, 1.0 + torch.randn(dim, generator=g) * 0.3
    inv_freq = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)]) if rot else None
    positions = torch.arange(5, 5 + tokens, dtype=torch.int32)
    token_seq = torch.zeros(tokens, dtype=torch.int32)
    cu_q, slots = torch.tensor([0, tokens], dtype=torch.int32), torch.tensor([0], dtype=torch.int32)
    table = torch.randperm(pages, generator=g).to(torch.int32).view(1, -1)
    results = []
    for device, module in (("cpu", refs), (DEV, ops)):
        kp = torch.zeros(pages, kv_heads, block, dim, dtype=dtype, device=device)
        vp = torch.zeros(pages, kv_heads, vdim, block, dtype=dtype, device=device)
        q = torch.zeros(tokens, heads * dim, dtype=dtype, device=device)
        moved = [None if t is None else t.to(device) for t in (qkv, bias, None, None, inv_freq, positions, token_seq, cu_q, slots, table)]
        module.conv_rope_norm_write(*moved, kp, vp, q, num_seqs=1, q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim,
                                    rotary_dim=rot, unit_norm_eps=1e-5, taps=0, norm_weight_q=wq.to(device), norm_weight_k=wk.to(device),
                                    norm_first=True)
        results.append((q, kp, vp))
    for got, want in zip(results[1], results[0]):
        close(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [4, 16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 24, 16), (6, 3, 64, 64), (8, 2, 128, 128), (2, 2, 10, 6), (3, 1, 80, 48)])
@pytest.mark.parametrize("window", [1, 7, 64, 150])
def test_one_key_at_the_window_s_edge_with_biases_by_distance(dtype, block_size, heads, kv_heads, dim, vdim, window):
    """Keys whose scores dominate sit just inside and just outside the window of the last token, of the
    portion's first token and of tokens between, at page borders and at the first position; a table of
    biases by distance of order one, laid out by distance with a last entry that serves every distance
    beyond: the attention kernels against the reference, for a prompt's portion behind cached keys and for
    single tokens."""
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
    pages = -(-length // block_size)
    perm = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    key_pages = torch.zeros(pages + 3, kv_heads, block_size, dim, dtype=dtype)
    value_pages = torch.zeros(pages + 3, kv_heads, vdim, block_size, dtype=dtype)
    for p in range(length):
        key_pages[perm[p // block_size], :, p % block_size] = k[p]
        value_pages[perm[p // block_size], :, :, p % block_size] = v[p]
    table = perm.view(1, -1)
    for span in (min(window, 40), window + 5):
        bias = torch.randn(heads, span, generator=g) * 2.0
        common = dict(q_heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, scale=0.4, window=window)
        portion = dict(num_seqs=1, max_q_len=length - cached, num_decode=0, max_ctx=length, **common)
        want = torch.zeros(length - cached, heads * vdim, dtype=dtype)
        refs.masked_attention(q[cached:].reshape(length - cached, -1), key_pages, value_pages, want, torch.tensor([0, length - cached]),
                              torch.tensor([length]), table, dist_bias=bias, **portion)
        out = torch.empty(length - cached, heads * vdim, dtype=dtype, device=DEV)
        ops.masked_attention(q[cached:].reshape(length - cached, -1).to(DEV), key_pages.to(DEV), value_pages.to(DEV), out,
                             torch.tensor([0, length - cached], dtype=torch.int32, device=DEV),
                             torch.tensor([length], dtype=torch.int32, device=DEV), table.to(DEV), dist_bias=bias.to(DEV), **portion)
        close(out, want, dtype)
        places = [0, block_size - 1, block_size, window - 1, window, min(window + 1, length - 1), cached, length - 1]
        n = len(places)
        singles = dict(num_seqs=n, max_q_len=1, num_decode=n, max_ctx=length, **common)
        want = torch.zeros(n, heads * vdim, dtype=dtype)
        refs.masked_attention(q[places].reshape(n, -1), key_pages, value_pages, want, torch.arange(n + 1),
                              torch.tensor([p + 1 for p in places]), table.expand(n, -1), dist_bias=bias, **singles)
        out = torch.empty(n, heads * vdim, dtype=dtype, device=DEV)
        ops.masked_attention(q[places].reshape(n, -1).to(DEV), key_pages.to(DEV), value_pages.to(DEV), out,
                             torch.arange(n + 1, dtype=torch.int32, device=DEV),
                             torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV), table.expand(n, -1).contiguous().to(DEV),
                             dist_bias=bias.to(DEV), **singles)
        close(out, want, dtype)


def latent_cache(length, row_dim, value_dim, block_size, dtype, g, loud=()):
    rows = torch.randn(length, row_dim, generator=g) * 0.5
    for far in loud:
        rows[far] *= 3.0
    rows = rows.to(dtype)
    pages = -(-length // block_size)
    perm = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)
    key_pages = torch.full((pages + 3, 1, block_size, row_dim), float("nan"), dtype=dtype)      # slots beyond the context may hold anything
    value_pages = torch.full((pages + 3, 1, value_dim, block_size), float("nan"), dtype=dtype)
    for p in range(length):
        key_pages[perm[p // block_size], 0, p % block_size] = rows[p]
        value_pages[perm[p // block_size], 0, :, p % block_size] = rows[p, :value_dim]
    return rows, key_pages, value_pages, perm.view(1, -1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [8, 16, 64])
@pytest.mark.parametrize("heads,row_dim,value_dim", [(4, 192, 128), (16, 96, 64), (3, 160, 128), (7, 320, 256), (20, 576, 512), (5, 40, 24), (2, 300, 280)])
def test_attention_over_a_latent_s_rows(dtype, block_size, heads, row_dim, value_dim):
    """One shared cache of rows read by every head: a prompt's portion behind cached rows (its rows span
    several blocks of 64 and end inside one), single tokens at the first position, at page borders and far
    back, with the keys cut into runs that are merged; loud rows at the first position and at page
    borders.  Sizes the matrix-core kernel is compiled for, and sizes it leaves to the vector-ALU kernel."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(heads + row_dim + block_size)
    length, cached = 270, 229
    _, key_pages, value_pages, table = latent_cache(length, row_dim, value_dim, block_size, dtype, g, loud=(0, block_size - 1, block_size, 63, 64, 228))
    q = (torch.randn(length, heads * row_dim, generator=g) * 0.5).to(dtype)
    n = length - cached
    shape = dict(heads=heads, row_dim=row_dim, value_dim=value_dim, scale=0.2)
    want = torch.zeros(n, heads * value_dim, dtype=dtype)
    refs.latent_attention(q[cached:], key_pages, value_pages, want, torch.tensor([0, n]), torch.tensor([length]), table, num_seqs=1, max_q_len=n, **shape)
    for splits in (None, 1, 3):
        out = torch.full((n, heads * value_dim), float("nan"), dtype=dtype, device=DEV)
        ops.latent_attention(q[cached:].to(DEV), key_pages.to(DEV), value_pages.to(DEV), out, torch.tensor([0, n], dtype=torch.int32, device=DEV),
                             torch.tensor([length], dtype=torch.int32, device=DEV), table.to(DEV), num_seqs=1, max_q_len=n, num_decode=0,
                             max_ctx=length, splits=splits, **shape)
        close(out, want, dtype, loose=3.0)
    places = [0, block_size - 1, block_size, 31, 32, 33, 127, 128, cached, length - 1]
    n = len(places)
    want = torch.zeros(n, heads * value_dim, dtype=dtype)
    refs.latent_attention(q[places], key_pages, value_pages, want, torch.arange(n + 1), torch.tensor([p + 1 for p in places]), table.expand(n, -1),
                          num_seqs=n, max_q_len=1, **shape)
    for splits in (None, 1, 2, 5):
        out = torch.full((n, heads * value_dim), float("nan"), dtype=dtype, device=DEV)
        ops.latent_attention(q[places].to(DEV), key_pages.to(DEV), value_pages.to(DEV), out, torch.arange(n + 1, dtype=torch.int32, device=DEV),
                             torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV), table.expand(n, -1).contiguous().to(DEV),
                             num_seqs=n, max_q_len=1, num_decode=n, max_ctx=length, splits=splits, **shape)
        close(out, want, dtype, loose=3.0)
    if dtype == torch.float32 or not ops.latent_attention_supported(dtype, row_dim, value_dim, block_size):
        # a cache of keys only: a row's first dims are its value
        out = torch.full((n, heads * value_dim), float("nan"), dtype=dtype, device=DEV)
        ops.latent_attention(q[places].to(DEV), key_pages.to(DEV), None, out, torch.arange(n + 1, dtype=torch.int32, device=DEV),
                             torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV), table.expand(n, -1).contiguous().to(DEV),
                             num_seqs=n, max_q_len=1, num_decode=n, max_ctx=length, **shape)
        close(out, want, dtype, loose=3.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim,turned", [(10, 12, 4, 4), (96, 128, 64, 64), (300, 512, 64, 32), (7, 20, 8, 0)])
def test_latent_norms_rotation_and_page_write(dtype, q_rank, kv_rank, rot_dim, turned):
    """The two bottlenecks' norms, the rotated part, the row into key pages and its first part into the
    transposed value pages; a reader that writes nothing; the query rows packed from the batched product
    and the rotated parts of q."""
    from forge_engine_amd.kernels import ops
    g = torch.Generator().manual_seed(q_rank + kv_rank)
    tokens, block, pages, heads, dim = 19, 8, 6, 3, 10
    x = torch.randn(tokens, q_rank + kv_rank + rot_dim + 2, generator=g) * 2.0
    wq, wkv = 1.0 + torch.randn(q_rank, generator=g) * 0.2, 1.0 + torch.randn(kv_rank, generator=g) * 0.2
    inv_freq = torch.tensor([80.0 ** (-2.0 * i / turned) for i in range(turned // 2)]) if turned else None
    positions = torch.arange(11, 11 + tokens, dtype=torch.int32)
    token_seq = torch.zeros(tokens, dtype=torch.int32)
    table = torch.randperm(pages, generator=g).to(torch.int32).view(1, -1)
    outs = []
    for device, module in (("cpu", refs), (DEV, ops)):
        kp = torch.zeros(pages, 1, block, kv_rank + rot_dim, dtype=dtype, device=device)
        vp = torch.zeros(pages, 1, kv_rank, block, dtype=dtype, device=device)
        cq = torch.zeros(tokens, q_rank, dtype=dtype, device=device)
        moved = [None if t is None else t.to(device) for t in (x, wq, wkv, inv_freq, positions, token_seq, table)]
        module.latent_norm_rope_write(*moved, kp, vp, cq, q_rank=q_rank, kv_rank=kv_rank, rot_dim=rot_dim, rotary_dim=turned, eps=1e-5,
                                      write_kv=True)
        only_q = torch.zeros(tokens, q_rank, dtype=dtype, device=device)
        module.latent_norm_rope_write(moved[0][:, :q_rank], moved[1], None, None, moved[4], moved[5], None, None, None, only_q, q_rank=q_rank,
                                      kv_rank=kv_rank, rot_dim=rot_dim, rotary_dim=turned, eps=1e-5, write_kv=False)
        q = (torch.randn(tokens, heads * (dim + rot_dim) + 4, generator=torch.Generator().manual_seed(1))).to(dtype).to(device)[:, :heads * (dim + rot_dim)]
        qa = torch.randn(heads, tokens, kv_rank, generator=torch.Generator().manual_seed(2)).to(dtype).to(device)
        packed = torch.zeros(tokens, heads, kv_rank + rot_dim, dtype=dtype, device=device)
        module.latent_query_pack(q, qa, moved[3], moved[4], packed, heads=heads, dim=dim, rot_dim=rot_dim, rotary_dim=turned, kv_rank=kv_rank)
        outs.append((kp, vp, cq, only_q, packed))
    for got, want in zip(outs[1], outs[0]):
        close(got, want, dtype)
    x3, w3 = torch.randn(tokens, heads, 12, generator=g).to(dtype), torch.randn(heads, 12, 9, generator=g).to(dtype)
    close(ops.heads_product(x3.to(DEV), w3.to(DEV)), refs.heads_product(x3, w3), dtype)


# ------------------------------------------------------------------ the model

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: du.write_model(raw, 31, tmp_path_factory.mktemp(f"dubizen_{name}")) for name, raw in CONFIGS.items()}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def expected(name, folder, cache, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in cache:
        cache[key] = du.plain_logits(folder, requests)
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
    worst = du.compare(got, expected(name, folders[name], plain_cache, requests), dtype)
    print(f"  worst difference {worst:.3e}", flush=True)


def sharpen(tensors):
    """Sharper attention: a key at a window's edge, and the first token of hundreds, reach the logits."""
    for name in tensors:
        if name.endswith((".mix.q.norm", ".mix.uq")):
            tensors[name] = (tensors[name].float() * 3.0).to(tensors[name].dtype)
        if name.endswith(".mix.rel"):
            tensors[name] = (tensors[name].float() * 2.0).to(tensors[name].dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_with_sharp_attention(dtype, tmp_path):
    """Prompts of several hundred tokens, longer than every window: whole, then the last 40 tokens one by
    one (across page borders and the windows' edges), then in portions, then three at once."""
    folder = du.write_model(du.MEDIUM, 32, tmp_path / "sharp", change=sharpen)
    requests = requests_of("M", 9, (500, 333, 129))
    want = du.plain_logits(folder, requests)
    for mode, trace in (("whole", ru.trace_whole(requests)), ("tail", ru.trace_tail(requests, 40)),
                        ("portions", ru.trace_portions(requests, sizes=(64, 17, 2, 130, 3, 48, 16, 2, 33), want_all=False)),
                        ("mixed", ru.trace_mixed(requests, 11, max_live=3))):
        print(f"sharp {mode} {dtype}: {len(trace.steps)} steps", flush=True)
        got = ru.run_trace(folder, dtype, trace, tmp_path / mode, block_size=16)
        du.compare(got, want, dtype, fraction=0.1, float32_factor=10.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_equal_eager_steps_and_long_decoding(dtype, folders):
    """A prompt and then 150 single tokens, two requests side by side: steps replayed from captured graphs
    against the same steps run eagerly, and both against the plain implementation."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["M"], dtype=dtype, device=DEV)
    requests = requests_of("M", 21, (160, 171))
    want = du.plain_logits(folders["M"], requests)
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
        du.compare(got, want, dtype, fraction=0.1)
    for key, row in results[True].items():
        torch.testing.assert_close(row, results[False][key], rtol=0, atol=0 if dtype == "float32" else 3e-2)      # captured steps cut the keys into other runs


def test_first_tokens_and_pages_used_again(folders):
    """Requests of one, two and a few tokens, one after the other through the same pages and the one state slot."""
    from forge_engine_amd.engine import ModelRunner, StepEntry, load_model
    _, model = load_model(folders["A"], dtype="float32", device=DEV)
    runner = ModelRunner(model, block_size=4, block_capacity=16, num_state_slots=1)
    cfg, weights = du.folder_weights(folders["A"])
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

    cfg, weights = du.folder_weights(folders["A"])

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
