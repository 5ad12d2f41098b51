"""Plain PyTorch references of every kernel entry point, with the same
signatures as ``forge_engine_amd.kernels.ops``.

Two uses: the GPU tests compare each HIP kernel alone with its reference here;
the CPU tests patch these in for the kernels (``install``) so that the step
function, the cache and the scheduler can be exercised without a GPU.  They
are test code: the product has no CPU path and never imports this file.
All arithmetic is float32 (float64 where noted), whatever the storage dtype.
"""

from __future__ import annotations

import torch


def embed_rows(ids, table, out, scale=1.0):
    out.copy_(table[ids.long()].float() * scale)
    return out


def add_rmsnorm(h, delta, weight, eps, out, rows=None, store_sum=True):
    if delta is not None and delta.dim() == 3:
        delta = delta.float().sum(0)
    if rows is not None:
        src = h[rows.long()]
        if delta is not None:
            src = src + delta[rows.long()].float()
    else:
        src = h if delta is None else h + delta.float()
        if delta is not None and store_sum:
            h.copy_(src)
    var = src.square().mean(dim=-1, keepdim=True)
    out.copy_((src * torch.rsqrt(var + eps) * weight).to(out.dtype))
    return out


def add_rows(h, delta):
    h += delta.float().sum(0) if delta.dim() == 3 else delta.float()
    return h


def swiglu(gate_up, out):
    inter = gate_up.shape[1] // 2
    g = gate_up[:, :inter].float()
    u = gate_up[:, inter:].float()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
    return out


def gemm_nt_f32(a, b, bias=None, out=None):
    y = a.double() @ b.double().T
    if bias is not None:
        y = y + bias.double()
    y = y.float()
    if out is None:
        return y
    out.copy_(y)
    return out


def linear(x, weight, bias=None, out_dtype=None):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype if out_dtype is None else out_dtype)


def linear_swiglu(x, gate_up_weight):
    inter = gate_up_weight.shape[0] // 2
    y = x.float() @ gate_up_weight.float().T
    g, u = y[:, :inter], y[:, inter:]
    return (g / (1.0 + torch.exp(-g)) * u).to(x.dtype)


def linear_update(x, weight, bias=None, stream=None):
    return linear(x, weight, bias, out_dtype=torch.float32)    # the stream is left to the caller's add


def gemm_skinny(x, weight, epilogue="bf16", tiles=0, waves=0, splits=1):
    if epilogue == "swiglu":
        return linear_swiglu(x, weight)
    return linear(x, weight, out_dtype=torch.float32 if epilogue == "f32" else torch.bfloat16)


def qk_norm_rope_write(qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table,
                       key_pages, value_pages, *, q_heads, kv_heads, head_dim, rotary_dim, eps,
                       write_kv=True):
    tokens = qkv.shape[0]
    heads = q_heads + (2 * kv_heads if write_kv else 0)
    x = qkv.view(tokens, heads, head_dim).float()

    def norm_rotate(y, w):
        if w is not None:
            y = y * torch.rsqrt(y.square().mean(-1, keepdim=True) + eps) * w
        if rotary_dim:
            half = rotary_dim // 2
            angle = positions.float().view(-1, 1, 1) * inv_freq.view(1, 1, half)
            cos, sin = angle.cos(), angle.sin()
            lo, hi = y[..., :half], y[..., half:rotary_dim]
            y = torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, y[..., rotary_dim:]), dim=-1)
        return y

    q = norm_rotate(x[:, :q_heads], q_weight)
    qkv.view(tokens, heads, head_dim)[:, :q_heads] = q.to(qkv.dtype)
    if not write_kv:
        return
    k = norm_rotate(x[:, q_heads:q_heads + kv_heads], k_weight).to(qkv.dtype)
    v = x[:, q_heads + kv_heads:].to(qkv.dtype)
    block_size = key_pages.shape[2]
    for t in range(tokens):
        pos = int(positions[t])
        page = int(block_table[int(token_seq[t]), pos // block_size])
        assert page >= 0, "token without a page"
        key_pages[page, :, pos % block_size] = k[t]
        value_pages[page, :, :, pos % block_size] = v[t]     # values are stored transposed: [D][slot]


def gather_pages(pages, table_row, length, block_size):
    """[kv_heads, length, D] from pages [blocks, kv_heads, block_size, D]; rows of
    pages that were given back (-1) are NaN so that any read of them shows."""
    kv_heads, head_dim = pages.shape[1], pages.shape[3]
    out = torch.full((kv_heads, length, head_dim), float("nan"))
    for start in range(0, length, block_size):
        page = int(table_row[start // block_size])
        count = min(block_size, length - start)
        if page >= 0:
            out[:, start:start + count] = pages[page, :, :count].float()
    return out


def paged_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, *, num_seqs, max_q_len,
                    q_heads, kv_heads, head_dim, scale, window=None, num_decode=None, max_ctx=None, splits=None):
    block_size = key_pages.shape[2]
    groups = q_heads // kv_heads
    key_pages, value_pages = key_pages.cpu(), value_pages.cpu()
    q_host, table, cu, ctxs = q.float().cpu(), block_table.cpu(), cu_q.cpu(), ctx_len.cpu()
    result = torch.zeros(out.shape, dtype=torch.float32)
    for s in range(num_seqs):
        q0, q1 = int(cu[s]), int(cu[s + 1])
        q_len, ctx = q1 - q0, int(ctxs[s])
        before = ctx - q_len
        keys = gather_pages(key_pages, table[s], ctx, block_size)
        values = gather_pages(value_pages.transpose(2, 3), table[s], ctx, block_size)
        queries = q_host[q0:q1, :q_heads * head_dim].reshape(q_len, q_heads, head_dim)
        for i in range(q_len):
            pos = before + i
            first = 0 if not window else max(0, pos - window + 1)
            for h in range(q_heads):
                kh = h // groups
                scores = (keys[kh, first:pos + 1] @ queries[i, h]) * scale
                probs = torch.softmax(scores, dim=0)
                result[q0 + i, h * head_dim:(h + 1) * head_dim] = probs @ values[kh, first:pos + 1]
    out.copy_(result.to(out.dtype))
    return out


def paged_attention_by_matrices(q, key_pages, value_pages, cu_q, ctx_len, block_table, *, q_heads, kv_heads,
                                head_dim, scale, window=None):
    """``paged_attention`` for long sequences: a whole (sequence, head) at a time as two float32
    matrix products with the causal (and window) mask between them, instead of a token at a time.
    The same formula; ``tests/test_kernel_policies.py`` holds the two against each other.  Returns float32."""
    block_size = key_pages.shape[2]
    groups = q_heads // kv_heads
    result = torch.zeros((q.shape[0], q_heads * head_dim), dtype=torch.float32)
    for s in range(ctx_len.numel()):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        q_len, ctx = q1 - q0, int(ctx_len[s])
        if q_len == 0:
            continue
        before = ctx - q_len
        keys = gather_pages(key_pages, block_table[s], ctx, block_size)
        values = gather_pages(value_pages.transpose(2, 3), block_table[s], ctx, block_size)
        position = before + torch.arange(q_len).view(-1, 1)
        key_index = torch.arange(ctx).view(1, -1)
        seen = key_index <= position
        if window:
            seen &= key_index > position - window
        keys, values = torch.nan_to_num(keys), torch.nan_to_num(values)   # pages given back lie outside every window
        for h in range(q_heads):
            queries = q[q0:q1, h * head_dim:(h + 1) * head_dim].float()
            scores = (queries @ keys[h // groups].T) * scale
            probs = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
            result[q0:q1, h * head_dim:(h + 1) * head_dim] = probs @ values[h // groups]
    return result


def argmax_rows(logits, tokens, status):
    for r in range(logits.shape[0]):
        row = logits[r]
        flags = 0
        if torch.isnan(row).any():
            flags |= 1
        if torch.isposinf(row).any():
            flags |= 2
        if not torch.isfinite(row).any():
            flags |= 4
        status[r] = flags
        tokens[r] = int(torch.argmax(row)) if not flags & 1 else 0


def philox_first_word(counter: int, key: int) -> int:
    """Philox4x32-10 with counter (lo, hi, 0, 0) and key (lo, hi); first word."""
    mask = 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [key & mask, (key >> 32) & mask]
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]
        p1 = 0xCD9E8D57 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + 0x9E3779B9) & mask, (k[1] + 0xBB67AE85) & mask]
    return c[0]


def uniform_from(counter: int, key: int) -> float:
    return (philox_first_word(counter, key) >> 8) / 16777216.0


def kept_after_filters(row, temperature, top_k, top_p, min_p):
    """(weights, kept) of one row in float64 after temperature, top-k, top-p, min-p in the order and
    with the rules of the reference (src/forge_engine/sampling.py:83-140): e_i = exp((x_i - max) / T);
    top-k keeps the k largest; top-p keeps a token if the probability of all larger ones, within what
    top-k left, is <= top_p; min-p keeps e_i >= min_p (the largest e is 1)."""
    # the logit as the kernel forms it, in float32: (max - x) * (1 / T); everything after it in float64
    y = (row.float().max() - row.float()) * torch.tensor(1.0, dtype=torch.float32).div(temperature)
    x = -y.double()
    e = torch.exp(x)
    kept = torch.ones_like(e, dtype=torch.bool)
    if top_k and top_k < len(row):
        kth = torch.topk(x, top_k).values[-1]
        kept &= x >= kth
    if top_p < 1.0:
        masked = torch.where(kept, e, torch.zeros_like(e))
        order = torch.argsort(x, descending=True, stable=True)
        before = masked[order].cumsum(0) - masked[order]
        keep_sorted = before <= top_p * masked.sum()
        by_p = torch.zeros_like(kept)
        by_p[order] = keep_sorted
        kept &= by_p
    if min_p > 0.0:
        kept &= e >= min_p
    return e, kept


def unpack_sample_params(params):
    """Rows of (temperature, top_k, top_p, min_p, seed, draw index) from the packed int32 words."""
    words = params.cpu().contiguous()
    floats = words.view(torch.float32)
    rows = []
    for r in range(words.shape[0]):
        low = [int(v) & 0xFFFFFFFF for v in words[r, 4:8]]
        rows.append((float(floats[r, 0]), int(words[r, 1]), float(floats[r, 2]), float(floats[r, 3]),
                     low[0] | (low[1] << 32), low[2] | (low[3] << 32)))
    return rows


def sample_filtered_rows(logits, params, tokens, status, any_top_k=True, any_top_p=True):
    """Arg-max (temperature 0), or the filters above and an inverse CDF in float64 over what they
    kept, in token order, with the same uniform as the kernel; the kernel's sums of 2^-40 steps may
    pick a neighbour when the target falls within rounding of a boundary (tests allow for that)."""
    for r, (temperature, top_k, top_p, min_p, seed, draw) in enumerate(unpack_sample_params(params)):
        row = logits[r]
        flags = 0
        if torch.isnan(row).any():
            flags |= 1
        if torch.isposinf(row).any():
            flags |= 2
        if not torch.isfinite(row).any():
            flags |= 4
        status[r] = flags
        if flags:
            tokens[r] = 0
            continue
        if not temperature > 0:
            tokens[r] = int(torch.argmax(row))
            continue
        e, kept = kept_after_filters(row, temperature, top_k, top_p, min_p)
        cdf = torch.where(kept, e, torch.zeros_like(e)).cumsum(0)
        target = uniform_from(draw, seed) * float(cdf[-1])
        pick = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
        tokens[r] = min(pick, logits.shape[1] - 1)


# ------------------------------------------------- ops on the stream, beside the matrix products

def cast_rows(h, dtype):
    return h if h.dtype == dtype else h.to(dtype)


def _sum_parts(update):
    return update.float().sum(0) if update.dim() == 3 else update.float()


def _unit(x, eps):
    return x * torch.rsqrt(x.square().mean(-1, keepdim=True) + eps)


def token_shift(x, weights, state, cu_q, token_seq, state_slots, *, num_seqs, out_dtype):
    xf = x.float()
    previous = torch.zeros_like(xf)
    for s in range(num_seqs):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        if b > a:
            previous[a] = state[int(state_slots[s])]
            previous[a + 1:b] = xf[a:b - 1]
    out = (xf[None] + (previous - xf)[None] * weights[:, None, :]).to(out_dtype)
    for s in range(num_seqs):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        if b > a:
            state[int(state_slots[s])] = xf[b - 1]
    return out


def rmsnorm_update(h, update, weight, eps, out=None):
    h += _unit(_sum_parts(update), eps) * weight
    if out is not None:
        out.copy_(h.to(out.dtype))
    return out


def rmsnorm_update_norm(h, update, weight, eps, next_weight, next_eps, out, rows=None):
    u = _sum_parts(update)
    v = h + _unit(u, eps) * weight
    if rows is None:
        h.copy_(v)
    else:
        v = v[rows.long()]
    out.copy_((_unit(v, next_eps) * next_weight).to(out.dtype))
    return out


def rmsnorm_mean(updates, weights, eps, out):
    total = torch.zeros_like(out)
    for index, update in enumerate(updates):
        total += _unit(_sum_parts(update), eps) * weights[index]
    out.copy_(total / len(updates))
    return out


def polynorm(z, coefficients, eps, out):
    y = z.float()
    a, b, c, e = (float(v) for v in coefficients)
    out.copy_((a * _unit(y, eps) + b * _unit(y * y, eps) + c * _unit(y * y * y, eps) + e).to(out.dtype))
    return out


def tanh_rows(x):
    x.copy_(torch.tanh(x.float()).to(x.dtype))
    return x


def _act(gate, act):
    if act == "silu":
        return gate * torch.sigmoid(gate)
    if act == "sigmoid":
        return torch.sigmoid(gate)
    return torch.ones_like(gate)


def head_norm_gate(o, weight, gate, out, *, heads, dim, eps, act="none", extra=0, floor=None):
    tokens = o.shape[0]
    y = o[..., :dim]
    if extra:
        y = y / (torch.maximum(o[..., dim].abs(), floor) + 1e-6)[..., None]
    y = _unit(y, eps)
    if weight is not None:
        y = y * (weight.view(heads, dim) if weight.numel() == heads * dim else weight.view(1, dim))
    y = y.reshape(tokens, heads * dim)
    if gate is not None:
        y = y * _act(gate.float(), act)
    out.copy_(y.to(out.dtype))
    return out


def add_bias(update, bias):
    if update.dim() == 3:
        update[0] += bias
    else:
        update += bias
    return update


def conv_rope_norm_write(qkv, bias, conv_weight, conv_state, inv_freq, positions, token_seq, cu_q, state_slots, block_table,
                         key_pages, value_pages, q_out, *, num_seqs, q_heads, kv_heads, head_dim, value_dim, rotary_dim,
                         unit_norm_eps, taps, v_from=None, v_mix=0.0, v_keep=None, norm_weight_q=None, norm_weight_k=None,
                         norm_first=False):
    tokens = qkv.shape[0]
    q_size, k_size, v_size = q_heads * head_dim, kv_heads * head_dim, kv_heads * value_dim
    channels = q_size + k_size + v_size
    u = qkv[:, :channels].float()
    if bias is not None:
        u = u + bias
    y = u.clone()
    if taps:
        for s in range(num_seqs):
            a, b = int(cu_q[s]), int(cu_q[s + 1])
            if b == a:
                continue
            if taps == 1:
                y[a:b] = u[a:b] * conv_weight[:, 0]
                continue
            slot = int(state_slots[s])
            history = torch.cat([conv_state[slot], u[a:b]])            # [taps - 1 + n, channels]
            y[a:b] = sum(history[j:j + b - a] * conv_weight[:, j] for j in range(taps))
            conv_state[slot] = history[-(taps - 1):]

    def rotate_norm(x, weight):
        if unit_norm_eps is not None and norm_first:
            x = _unit(x, unit_norm_eps) * (1.0 if weight is None else weight)
        if rotary_dim:
            half = rotary_dim // 2
            angle = positions.float().view(-1, 1, 1) * inv_freq.view(1, 1, half)
            cos, sin = angle.cos(), angle.sin()
            lo, hi = x[..., :half], x[..., half:rotary_dim]
            x = torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, x[..., rotary_dim:]), dim=-1)
        if unit_norm_eps is not None and not norm_first:
            x = _unit(x, unit_norm_eps) * (1.0 if weight is None else weight)
        return x

    q = rotate_norm(y[:, :q_size].view(tokens, q_heads, head_dim), norm_weight_q)
    k = rotate_norm(y[:, q_size:q_size + k_size].view(tokens, kv_heads, head_dim), norm_weight_k).to(qkv.dtype)
    v = y[:, q_size + k_size:]
    if v_from is not None:
        v = (1.0 - v_mix) * v + v_mix * v_from.float()
    v = v.view(tokens, kv_heads, value_dim).to(qkv.dtype)
    if v_keep is not None:
        v_keep.copy_(v.reshape(tokens, v_size))
    q_out.copy_(q.reshape(tokens, q_size).to(q_out.dtype))
    block_size = key_pages.shape[2]
    for t in range(tokens):
        pos = int(positions[t])
        page = int(block_table[int(token_seq[t]), pos // block_size])
        assert page >= 0, "token without a page"
        key_pages[page, :, pos % block_size] = k[t]
        value_pages[page, :, :, pos % block_size] = v[t]


def masked_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, *, num_seqs, max_q_len, q_heads, kv_heads,
                     head_dim, value_dim, scale, window=None, chunk=None, sink=None, gate=None, num_decode=None, max_ctx=None,
                     softcap=None, head_gate=False, slopes=None, dist_bias=None):
    block_size = key_pages.shape[2]
    groups = q_heads // kv_heads
    for s in range(num_seqs):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        ctx = int(ctx_len[s])
        if b == a:
            continue
        keys = gather_pages(key_pages, block_table[s], ctx, block_size)                         # [kv, ctx, D]
        if value_pages is None:      # a cache of keys only: a key's first dims are its value
            values = keys[..., :value_dim]
        else:
            values = gather_pages(value_pages.transpose(2, 3), block_table[s], ctx, block_size)     # [kv, ctx, Dv]
        for i in range(b - a):
            p = ctx - (b - a) + i
            first = 0
            if window is not None:
                first = max(first, p - window + 1)
            if chunk is not None:
                first = max(first, p // chunk * chunk)
            for h in range(q_heads):
                g = h // groups
                qv = q[a + i, h * head_dim:(h + 1) * head_dim].float()
                scores = (keys[g, first:p + 1] @ qv) * scale
                if softcap is not None:
                    scores = softcap * torch.tanh(scores / softcap)
                if slopes is not None:
                    scores = scores - slopes[h] * (p - torch.arange(first, p + 1, device=scores.device)).float()
                if dist_bias is not None:
                    distance = (p - torch.arange(first, p + 1, device=scores.device)).clamp(max=dist_bias.shape[1] - 1)
                    scores = scores + dist_bias[h, distance]
                top = scores.max()
                if sink is not None:
                    top = torch.maximum(top, sink[h])
                e = torch.exp(scores - top)
                denom = e.sum() + (torch.exp(sink[h] - top) if sink is not None else 0.0)
                o = (e / denom) @ values[g, first:p + 1]
                if gate is not None and head_gate:
                    o = o * torch.sigmoid(gate[a + i, h].float())
                elif gate is not None:
                    o = o * torch.sigmoid(gate[a + i, h * value_dim:(h + 1) * value_dim].float())
                out[a + i, h * value_dim:(h + 1) * value_dim] = o.to(out.dtype)
    return out


def linear_recurrence(q, k, v, out, state, cu_q, state_slots, *, num_seqs, max_q_len, heads, key_dim, value_dim,
                      decay=None, decay_kind="none", decay_bias=None, tau=1.0, head_decay=None, in_scale=None,
                      q_scale=1.0, bonus=None, ones_column=False):
    tokens = q.shape[0]
    qf = q.float().reshape(tokens, heads, key_dim) * q_scale
    kf = k.float().reshape(tokens, heads, key_dim)
    vf = v.float().reshape(tokens, heads, value_dim)
    if ones_column:
        vf = torch.cat([vf, torch.ones(tokens, heads, 1)], dim=-1)
    a = torch.ones(tokens, heads, key_dim)
    if decay_kind == "exp_neg_exp":
        a = torch.exp(-torch.exp(decay + decay_bias)).view(tokens, heads, key_dim)
    elif decay_kind == "sigmoid_root":
        a = torch.exp(torch.nn.functional.logsigmoid(decay + decay_bias) / tau).view(tokens, heads, key_dim)
    if head_decay is not None:
        a = a * head_decay[..., None]
    b = torch.ones(tokens, heads) if in_scale is None else in_scale
    u = None if bonus is None else bonus.reshape(heads, key_dim)
    for s in range(num_seqs):
        first, last = int(cu_q[s]), int(cu_q[s + 1])
        if last == first:
            continue
        slot = int(state_slots[s])
        S = state[slot].transpose(1, 2).clone()               # [heads, key, value]
        for t in range(first, last):
            kv = b[t][:, None, None] * kf[t][:, :, None] * vf[t][:, None, :]
            if u is not None:
                out[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, qf[t])
                S = a[t][:, :, None] * S + kv
            else:
                S = a[t][:, :, None] * S + kv
                out[t] = torch.einsum("hkv,hk->hv", S, qf[t])
        state[slot] = S.transpose(1, 2)
    return out


def mlstm_gate_scan(gates, bias, cap, maximum, cu_q, state_slots, out, *, num_seqs, heads):
    g = gates + bias
    gi = cap * torch.tanh(g[:, :heads] / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(g[:, heads:] / cap))
    for s in range(num_seqs):
        first, last = int(cu_q[s]), int(cu_q[s + 1])
        if last == first:
            continue
        m = maximum[int(state_slots[s])].clone()
        for t in range(first, last):
            m_new = torch.maximum(gf[t] + m, gi[t])
            out[0, t] = torch.exp(gf[t] + m - m_new)
            out[1, t] = torch.exp(gi[t] - m_new)
            out[2, t] = torch.exp(-m_new)
            m = m_new
        maximum[int(state_slots[s])] = m
    return out


def hyper_norm(streams, update, mix, share, read, weight, bias, eps, out, rows=None, store=True, rms=False):
    count = streams.shape[0]
    x = streams
    if update is not None:
        y = _sum_parts(update)
        m = torch.eye(count) if mix is None else mix
        sh = torch.ones(count) if share is None else share
        x = torch.einsum("sr,stw->rtw", m, streams) + sh[:, None, None] * y[None]
        if store and rows is None:
            streams.copy_(x)
    if out is None:
        return None
    u = x.sum(0) if read is None else torch.einsum("s,stw->tw", read, x)
    if rows is not None:
        u = u[rows.long()]
    if rms:
        z = u * torch.rsqrt(u.square().mean(-1, keepdim=True) + eps) * weight
    else:
        centred = u - u.mean(-1, keepdim=True)
        z = centred * torch.rsqrt(centred.square().mean(-1, keepdim=True) + eps) * weight
    if bias is not None:
        z = z + bias
    out.copy_(z.to(out.dtype))
    return out


def embed_token_pairs(ids, table, pair_table, positions, token_seq, cu_q, state_slots, previous, out, *, num_seqs, buckets,
                      mul_prev, mul_cur):
    for t in range(ids.numel()):
        cur = int(ids[t])
        if int(positions[t]) == 0:
            row = buckets
        else:
            s = int(token_seq[t])
            prev = int(ids[t - 1]) if t > int(cu_q[s]) else int(previous[int(state_slots[s]), 0])
            row = (prev * mul_prev + cur * mul_cur) % buckets
        out[t] = table[cur].float() + pair_table[row].float()
    for s in range(num_seqs):
        if int(cu_q[s + 1]) > int(cu_q[s]):
            previous[int(state_slots[s]), 0] = ids[int(cu_q[s + 1]) - 1]
    return out


def scale_rows(x, factor):
    return x.mul_(factor)


def whole_norm_rope_write(qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table, key_pages, value_pages, q_out, *,
                          q_heads, kv_heads, head_dim, value_dim, rotary_dim, eps, magnitude=1.0, write_kv=True):
    tokens = qkv.shape[0]
    q_size, k_size, v_size = q_heads * head_dim, kv_heads * head_dim, kv_heads * value_dim

    def prepare(x, weight, heads):
        x = x.float()
        x = (x * torch.rsqrt(x.square().mean(-1, keepdim=True) + eps) * weight).view(tokens, heads, head_dim)
        if rotary_dim:
            half = rotary_dim // 2
            angle = positions.float().view(-1, 1, 1) * inv_freq.view(1, 1, half)
            cos, sin = angle.cos() * magnitude, angle.sin() * magnitude
            lo, hi = x[..., :half], x[..., half:rotary_dim]
            x = torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, x[..., rotary_dim:]), dim=-1)
        return x

    q_out.copy_(prepare(qkv[:, :q_size], q_weight, q_heads).reshape(tokens, q_size).to(q_out.dtype))
    if not write_kv:
        return
    k = prepare(qkv[:, q_size:q_size + k_size], k_weight, kv_heads).to(qkv.dtype)
    v = qkv[:, q_size + k_size:q_size + k_size + v_size].view(tokens, kv_heads, value_dim)
    block_size = key_pages.shape[2]
    for t in range(tokens):
        pos = int(positions[t])
        page = int(block_table[int(token_seq[t]), pos // block_size])
        assert page >= 0, "token without a page"
        key_pages[page, :, pos % block_size] = k[t]
        value_pages[page, :, :, pos % block_size] = v[t]


def moe_route(x, router_weight, router_bias, top, scoring="softmax"):
    z = x.float() @ router_weight.float().T
    if router_bias is not None:
        z = z + router_bias
    best = torch.topk(z, top, dim=-1)
    weights = torch.sigmoid(best.values) if scoring == "sigmoid" else torch.softmax(best.values, dim=-1)
    return best.indices.to(torch.int32), weights


def _gated(g, u, limit, alpha, form="bounded"):
    if form == "silu":
        return g * torch.sigmoid(g) * u
    g = g.clamp(max=limit)
    return g * torch.sigmoid(alpha * g) * (u.clamp(-limit, limit) + 1.0)


def moe_experts(x, chosen, weights, gate_up, down, out, *, limit=0.0, alpha=1.0, extra=None, form="bounded", weight_input=False):
    inner = gate_up.shape[1] // 2
    for t in range(x.shape[0]):
        for k in range(chosen.shape[1]):
            e = int(chosen[t, k])
            gu = gate_up[e].float() @ x[t].float()
            if weight_input:
                gu = gu * weights[t, k]
            act = _gated(gu[:inner], gu[inner:], limit, alpha, form).to(x.dtype).float()
            out[k, t] = (1.0 if weight_input else weights[t, k]) * (down[e].float() @ act)
    if extra is not None:
        out[0] += _sum_parts(extra)
    return out


def linear_gated(x, gate_up_weight, *, limit, alpha):
    gu = linear(x, gate_up_weight).float()
    inner = gu.shape[1] // 2
    return _gated(gu[:, :inner], gu[:, inner:], limit, alpha).to(x.dtype)


def relu_squared(x):
    return torch.relu(x.float()).square().to(x.dtype)


def causal_conv_act(u, weight, bias, state, token_seq, cu_q, state_slots, *, num_seqs, act="silu"):
    channels, taps = weight.shape
    rows = u[:, :channels].float()
    out = torch.empty((u.shape[0], channels), dtype=u.dtype, device=u.device)
    for s in range(num_seqs):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        if b == a:
            continue
        if taps > 1:
            slot = int(state_slots[s])
            history = torch.cat([state[slot], rows[a:b]])
            state[slot] = history[-(taps - 1):]
        else:
            history = rows[a:b]
        y = sum(history[j:j + b - a] * weight[:, j] for j in range(taps))
        if bias is not None:
            y = y + bias
        if act == "silu":
            y = y * torch.sigmoid(y)
        out[a:b] = y.to(out.dtype)
    return out


def selective_scan(x, dt_lin, dt_bias, a, bc, d, z, state, cu_q, state_slots, *, num_seqs):
    channels, states = a.shape
    out = torch.empty_like(x)
    dt = torch.nn.functional.softplus((dt_lin + dt_bias).double())
    for s in range(num_seqs):
        lo, hi = int(cu_q[s]), int(cu_q[s + 1])
        if hi == lo:
            continue
        slot = int(state_slots[s])
        memory = state[slot].double()
        for t in range(lo, hi):
            xt = x[t].double()
            memory = torch.exp(dt[t][:, None] * a.double()) * memory + (dt[t] * xt)[:, None] * bc[t, :states].double()[None, :]
            y = memory @ bc[t, states:2 * states].double() + d.double() * xt
            zt = z[t, :channels].double()
            out[t] = (y * zt * torch.sigmoid(zt)).to(out.dtype)
        state[slot] = memory.float()
    return out


def layernorm_update(h, update, weight, eps, factor=1.0, out=None):
    u = _sum_parts(update)
    centred = u - u.mean(-1, keepdim=True)
    h += factor * centred * torch.rsqrt(centred.square().mean(-1, keepdim=True) + eps) * weight
    if out is not None:
        out.copy_(h.to(out.dtype))
    return out


def activate(x, kind):
    z = x.float()
    if kind == "relu_squared":
        y = torch.relu(z).square()
    elif kind == "gelu":
        y = 0.5 * z * (1.0 + torch.erf(z * 0.7071067811865476))
    elif kind == "gelu_tanh":
        y = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))
    else:
        raise ValueError(kind)
    return y.to(x.dtype)


def gate_rows(update, logits, column):
    update *= torch.sigmoid(logits[:, column]).view(-1, 1)
    return update


def _turn(r, positions, inv_freq, rotary_dim):
    """r [T, ..., n]: its first rotary_dim dims rotated, dim i with dim i + rotary_dim / 2."""
    if not rotary_dim:
        return r
    half = rotary_dim // 2
    angle = positions.float().view(-1, *([1] * (r.dim() - 2)), 1) * inv_freq.view(*([1] * (r.dim() - 1)), half)
    cos, sin = angle.cos(), angle.sin()
    lo, hi = r[..., :half], r[..., half:rotary_dim]
    return torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, r[..., rotary_dim:]), dim=-1)


def latent_norm_rope_write(x, q_weight, kv_weight, inv_freq, positions, token_seq, block_table, key_pages, value_pages, cq_out, *,
                           q_rank, kv_rank, rot_dim, rotary_dim, eps, write_kv):
    x = x.float()
    cq_out.copy_((_unit(x[:, :q_rank], eps) * q_weight).to(cq_out.dtype))
    if not write_kv:
        return cq_out
    latent = _unit(x[:, q_rank:q_rank + kv_rank], eps) * kv_weight
    turned = _turn(x[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim], positions, inv_freq, rotary_dim)
    rows = torch.cat((latent, turned), dim=-1).to(key_pages.dtype)
    block_size = key_pages.shape[2]
    for t in range(x.shape[0]):
        pos = int(positions[t])
        page = int(block_table[int(token_seq[t]), pos // block_size])
        assert page >= 0, "token without a page"
        key_pages[page, 0, pos % block_size] = rows[t]
        if value_pages is not None:
            value_pages[page, 0, :, pos % block_size] = rows[t, :kv_rank]
    return cq_out


def latent_query_pack(q, qa, inv_freq, positions, out, *, heads, dim, rot_dim, rotary_dim, kv_rank):
    tokens = q.shape[0]
    turned = _turn(q.view(tokens, heads, dim + rot_dim)[:, :, dim:].float(), positions, inv_freq, rotary_dim)
    out[:, :, :kv_rank] = qa.transpose(0, 1)
    out[:, :, kv_rank:] = turned.to(out.dtype)
    return out


def latent_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, *, num_seqs, max_q_len, heads, row_dim, value_dim,
                     scale, num_decode=None, max_ctx=None, splits=None):
    block_size = key_pages.shape[2]
    for s in range(num_seqs):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        ctx = int(ctx_len[s])
        if b == a:
            continue
        rows = gather_pages(key_pages, block_table[s], ctx, block_size)[0]            # [ctx, row_dim]
        values = rows[:, :value_dim] if value_pages is None else gather_pages(value_pages.transpose(2, 3), block_table[s], ctx, block_size)[0]
        for i in range(b - a):
            p = ctx - (b - a) + i
            queries = q[a + i].float().view(heads, row_dim)
            weights = torch.softmax(queries @ rows[:p + 1].T * scale, dim=-1)         # [heads, p + 1]
            out[a + i] = (weights @ values[:p + 1]).reshape(-1).to(out.dtype)
    return out


def heads_product(x, weight):
    return torch.einsum("thk,hkn->htn", x.float(), weight.float()).to(x.dtype)


def moe_route_grouped(x, router_weight, correction, *, experts, top, groups=1, keep=1, scale=1.0):
    logits = x.float() @ router_weight.float().T
    scores = torch.softmax(logits[:, :experts], dim=-1)
    choice = scores if correction is None else scores + correction
    if keep < groups:
        best = choice.view(-1, groups, experts // groups).max(-1).values                         # [T, groups]
        order = torch.argsort(best, dim=-1, descending=True, stable=True)[:, :keep]
        kept = torch.zeros_like(best, dtype=torch.bool).scatter_(1, order, True)
        choice = choice.masked_fill(~kept.repeat_interleave(experts // groups, dim=1), float("-inf"))
    chosen = torch.argsort(choice, dim=-1, descending=True, stable=True)[:, :top]
    own = scores.gather(1, chosen)
    weights = own / (own.sum(-1, keepdim=True) + 1e-20) * scale
    return chosen.to(torch.int32), weights, logits


def decode_prepare_supported(*args, **kwargs):
    return False        # on the CPU a step of single tokens takes the two references below in turn


def linear_in_parts(x, weight):
    return None


# Key splits of the bfloat16 decode attention that the GPU tests launch (every count the kernel takes:
# 1 to 4, 5 to 8 and 9 to 16 merge with all loads in one round, 17 to 64 in a loop)
DECODE_SPLITS_TESTED = tuple(range(1, 65))


NAMES = ("decode_prepare_supported", "linear_in_parts", "embed_rows", "add_rmsnorm", "add_rows", "swiglu", "gemm_nt_f32", "linear", "linear_update", "linear_swiglu", "gemm_skinny",
         "qk_norm_rope_write", "paged_attention", "argmax_rows", "sample_filtered_rows",
         "cast_rows", "add_bias", "token_shift", "rmsnorm_update", "rmsnorm_mean", "polynorm", "tanh_rows", "head_norm_gate",
         "conv_rope_norm_write", "masked_attention", "linear_recurrence", "mlstm_gate_scan",
         "hyper_norm", "embed_token_pairs", "scale_rows", "whole_norm_rope_write", "moe_route", "moe_experts", "linear_gated",
         "relu_squared", "causal_conv_act", "selective_scan", "rmsnorm_update_norm", "layernorm_update", "activate", "gate_rows",
         "latent_norm_rope_write", "latent_query_pack", "latent_attention", "heads_product", "moe_route_grouped")


def install(monkeypatch):
    """Patch the references in for the HIP kernels (CPU tests only)."""
    from forge_engine_amd.kernels import ops

    for name in NAMES:
        monkeypatch.setattr(ops, name, globals()[name])
