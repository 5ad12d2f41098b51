"""Grouped-query causal self-attention over the paged cache.

In order (reference: src/forge_engine/qwen3.py:132-207): q, k, v projections
(one fused product here); RMSNorm of each q and k head over the head dim with a
weight shared by all heads, before the rotation; rotary positions; attention of
each query head h over the keys of kv head h // G with scale head_dim^-0.5 and
the causal mask; output projection.  The keys and values of the step's tokens
go into their pages first, and attention then reads everything through the
block table, so a step may hold any portion of any request.

Options beside that (each off by default, constants as parameters):
``value_dim`` (values of another width than keys); ``conv_taps`` (a short causal
convolution over time on every channel of q, k and v, straight after the projection:
``y_t = sum_j c[:, j] * u_(t - taps + 1 + j)``, the last taps - 1 projected rows of a request kept
as fixed-size state); ``unit_norm_eps`` (after the rotation, q and k heads are divided by their
root mean square, no weight); ``chunk`` (token i sees key j <= i only if both lie in the same
run of ``chunk`` positions counted from position 0); ``sink`` (a learned number per query head
whose exponential joins the softmax's denominator, without key or value); ``output_gate``
(the concatenated heads times sigmoid(W_g x) before the output projection; with ``head_gate`` W_g has
one row per query head and the whole head is multiplied by that one number); ``whole_norm_eps``
(q, and k, divided by the root mean square over the whole projection, all heads at once, times a
weight of that size, before the rotation); ``softcap`` (scores, after the scale, bounded as
``cap * tanh(score / cap)``); ``own_kv`` False (the layer has no k and v tensors at all and is only
ever scheduled to read another call's cache); ``names`` (what the tensors are called in the
checkpoint); ``output_bias`` (whether the output projection has a bias; by default as ``bias`` says, False
gives biases on q, k and v alone); ``fixed_sink`` (a number that joins every head's softmax as a
score without key or value: 0 puts a one into the denominator); ``distance_slope_bits`` (c: head h's
score of key j loses ``2^(-c (h + 1) / H) * (i - j)``, H heads, after the scale); ``value_mix``
("source": the layer leaves its values of the step's tokens for later layers; "blend": its values
become ``(1 - m) v + m v_source`` with m a scalar tensor of the layer, before they are cached);
``distance_bias`` (``{"rows": B, "reach": D}``: a learned table [B, H] whose row ``bucket(i - j)`` is
added to head h's score of key j after the scale, which does not multiply it; ``bucket(n) = n`` below
B / 2, else ``min(B - 1, B / 2 + floor(ln(n / (B / 2)) / ln(D / (B / 2)) * (B - B / 2)))``: one row a distance
at first, logarithmic steps beyond, the last row from distance D on; the rows are laid out by distance
once, when the table is loaded); ``qk_norm_eps`` on the general path (the weighted RMS norm of every q
and k head, before the rotation, in the kernel that writes the pages);
``force_general`` (take the general path whatever the options).  A position part may scale its
cosines and sines (``magnitude``).  With any of them the step takes the general path:
one product for q, k, v (and the gate), one kernel for convolution, rotation, norms and the
page write, the masked attention kernel, the gate, the output projection.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, FixedState, PagedKV
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec, build_part
from .plan import PartSpec


class GroupedQueryAttention(Mixer):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, num_heads: int,
                 num_kv_heads: int, head_dim: int, position: PartSpec, qk_norm_eps: float | None = None,
                 bias: bool = False, window: int | None = None, scale: float | None = None,
                 value_dim: int | None = None, conv_taps: int = 0, unit_norm_eps: float | None = None,
                 chunk: int | None = None, sink: bool = False, output_gate: bool = False,
                 head_gate: bool = False, whole_norm_eps: float | None = None, softcap: float | None = None,
                 own_kv: bool = True, names: dict[str, str] | None = None, output_bias: bool | None = None,
                 fixed_sink: float | None = None, distance_slope_bits: float | None = None,
                 value_mix: str | None = None, value_mix_key: str = "values", force_general: bool = False,
                 bias_init: str = "zeros", distance_bias: dict | None = None) -> None:
        super().__init__(ctx, prefix)
        self.bias_init = bias_init      # how random models draw the biases of q, k and v ("small": so that they show)
        if num_heads % num_kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        if head_dim % 2 or not 2 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim} is not supported: even sizes from 2 to 256")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        self.v_size = num_kv_heads * self.value_dim
        self.out_size = num_heads * self.value_dim
        self.conv_taps = int(conv_taps)
        self.unit_norm_eps = unit_norm_eps
        self.chunk = chunk
        self.sink = sink
        self.output_gate = output_gate or head_gate
        self.head_gate = head_gate
        self.whole_norm_eps = whole_norm_eps
        self.softcap = None if softcap is None else float(softcap)
        self.own_kv = own_kv
        self.gate_size = 0 if not self.output_gate else (num_heads if head_gate else self.out_size)
        self.output_bias = bool(bias) if output_bias is None else bool(output_bias)
        self.fixed_sink = None if fixed_sink is None else float(fixed_sink)
        self.distance_slope_bits = None if distance_slope_bits is None else float(distance_slope_bits)
        if value_mix not in (None, "source", "blend"):
            raise ValueError(f"value_mix must be 'source' or 'blend', not {value_mix!r}")
        if sink and fixed_sink is not None:
            raise ValueError("a learned sink and a fixed one exclude each other")
        if self.output_bias and not bias:
            raise ValueError("a bias on the output projection comes with biases on q, k and v")
        self.value_mix, self.value_mix_key = value_mix, value_mix_key
        self.distance_bias = None
        if distance_bias is not None:
            rows, reach = int(distance_bias["rows"]), float(distance_bias["reach"])
            if rows < 2 or not reach > rows // 2:
                raise ValueError(f"a table of biases by distance needs two rows or more and a reach beyond half its rows, not {rows} and {reach}")
            self.distance_bias = (rows, reach)
        self.bias_table: Tensor | None = None       # as loaded [rows, heads]; by distance [heads, span] after finalize
        self.mix_weight: float | None = None
        self.slopes: Tensor | None = None
        if whole_norm_eps is not None and (self.conv_taps or unit_norm_eps is not None or bias):
            raise ValueError("a norm over the whole projection is not combined with convolutions, unit norms or biases")
        if not own_kv and whole_norm_eps is None:
            raise ValueError("a layer without keys and values of its own takes the path of the whole-projection norm")
        if self.conv_taps < 0:
            raise ValueError("a short convolution has at least one tap (0: none)")
        if chunk is not None and (chunk < 1 or window is not None):
            raise ValueError("chunk must be positive and cannot be combined with a window")
        # the general path: anything the fused kernels of the plain arrangement do not know
        self.general = bool(self.value_dim != head_dim or self.conv_taps or unit_norm_eps is not None
                            or chunk is not None or sink or self.output_gate or whole_norm_eps is not None
                            or softcap is not None or not own_kv or fixed_sink is not None
                            or distance_slope_bits is not None or value_mix is not None
                            or self.output_bias != bool(bias) or force_general or distance_bias is not None)
        if (value_mix is not None or fixed_sink is not None or distance_slope_bits is not None) and whole_norm_eps is not None:
            raise ValueError("value mixing, fixed sinks and distance slopes are not combined with the whole-projection norm")
        if self.general and qk_norm_eps is not None and (whole_norm_eps is not None or unit_norm_eps is not None):
            raise ValueError("weighted q/k norms before the rotation are not combined with another norm of q and k")
        if distance_bias is not None and whole_norm_eps is not None:
            raise ValueError("biases by distance are not combined with the whole-projection norm")
        self.names = dict(self.DEFAULT_NAMES, **(names or {}))
        self.qk_norm_eps = qk_norm_eps
        self.bias = bias
        self.window = window
        self.scale = head_dim ** -0.5 if scale is None else float(scale)
        self.position = build_part("position", position, ctx)
        self.conv_channels = self.q_size + self.kv_size + self.v_size
        if not own_kv:
            self.conv_channels = self.q_size
        width = self.conv_channels + self.gate_size
        self._rows = {"q": (0, self.q_size)}
        if own_kv:
            self._rows.update({"k": (self.q_size, self.kv_size), "v": (self.q_size + self.kv_size, self.v_size)})
        if self.output_gate:
            self._rows["gate"] = (self.conv_channels, self.gate_size)
        self._width = width
        self.conv_weight: Tensor | None = None
        self.sink_weight: Tensor | None = None
        self.qkv_weight: Tensor | None = None
        self.qkv_bias: Tensor | None = None
        self.o_weight: Tensor | None = None
        self.o_bias: Tensor | None = None
        self.q_norm: Tensor | None = None
        self.k_norm: Tensor | None = None

    # ------------------------------------------------------------ tensors
    DEFAULT_NAMES = {
        "q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
        "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
        "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
        "q_conv": "q_proj.conv", "k_conv": "k_proj.conv", "v_conv": "v_proj.conv",
        "sink": "sink", "gate": "gate_proj.weight", "value_mix": "value_mix", "distance_bias": "distance_bias",
    }

    def param_specs(self):
        n = {key: self.name(leaf) for key, leaf in self.names.items()}
        specs = {
            n["q"]: ParamSpec((self.q_size, self.hidden_size)),
        }
        if self.own_kv:
            specs[n["k"]] = ParamSpec((self.kv_size, self.hidden_size))
            specs[n["v"]] = ParamSpec((self.v_size, self.hidden_size))
        specs[n["o"]] = ParamSpec((self.hidden_size, self.out_size))
        if self.whole_norm_eps is not None:
            specs[n["q_norm"]] = ParamSpec((self.q_size,), kind="vector", init="norm")
            if self.own_kv:
                specs[n["k_norm"]] = ParamSpec((self.kv_size,), kind="vector", init="norm")
        if self.bias:
            drawn = self.bias_init
            specs[n["q_bias"]] = ParamSpec((self.q_size,), kind="vector", init=drawn)
            specs[n["k_bias"]] = ParamSpec((self.kv_size,), kind="vector", init=drawn)
            specs[n["v_bias"]] = ParamSpec((self.v_size,), kind="vector", init=drawn)
            if self.output_bias:
                specs[n["o_bias"]] = ParamSpec((self.hidden_size,), kind="vector", init="zeros")
        if self.qk_norm_eps is not None:
            specs[n["q_norm"]] = ParamSpec((self.head_dim,), kind="vector", init="norm")
            specs[n["k_norm"]] = ParamSpec((self.head_dim,), kind="vector", init="norm")
        if self.conv_taps:
            specs[n["q_conv"]] = ParamSpec((self.q_size, self.conv_taps), kind="vector", init="taps")
            specs[n["k_conv"]] = ParamSpec((self.kv_size, self.conv_taps), kind="vector", init="taps")
            specs[n["v_conv"]] = ParamSpec((self.v_size, self.conv_taps), kind="vector", init="taps")
        if self.sink:
            specs[n["sink"]] = ParamSpec((self.num_heads,), kind="vector", init="unit")
        if self.distance_bias is not None:
            specs[n["distance_bias"]] = ParamSpec((self.distance_bias[0], self.num_heads), kind="vector", init="unit")
        if self.output_gate:
            specs[n["gate"]] = ParamSpec((self.gate_size, self.hidden_size))
        if self.value_mix is not None:      # a scalar; the source layer's is never read
            specs[n["value_mix"]] = ParamSpec((), kind="vector", init="uniform", optional=self.value_mix == "source")
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        local = name[len(self.prefix) + 1:] if self.prefix else name
        key = next((k for k, leaf in self.names.items() if leaf == local), None)
        if key in self._rows:
            start, size = self._rows[key]
            if self.qkv_weight is None:  # the projections share one matrix: one product per step
                self.qkv_weight = torch.empty((self._width, self.hidden_size), dtype=tensor.dtype,
                                              device=tensor.device)
            if tensor.dtype != self.qkv_weight.dtype:
                raise ValueError(f"{name}: the projections of one input must be stored in one dtype")
            self.qkv_weight[start:start + size].copy_(tensor)
        elif key in ("q_bias", "k_bias", "v_bias"):
            start, size = self._rows[key[0]]
            if self.qkv_bias is None:
                self.qkv_bias = torch.zeros(self._width, dtype=torch.float32, device=tensor.device)
            self.qkv_bias[start:start + size].copy_(tensor)
        elif key in ("q_conv", "k_conv", "v_conv"):
            start, size = self._rows[key[0]]
            if self.conv_weight is None:
                self.conv_weight = torch.zeros((self.conv_channels, self.conv_taps), dtype=torch.float32,
                                               device=tensor.device)
            self.conv_weight[start:start + size].copy_(tensor)
        elif key == "o":
            self.o_weight = tensor
        elif key == "o_bias":
            self.o_bias = tensor
        elif key == "q_norm":
            self.q_norm = tensor
        elif key == "k_norm":
            self.k_norm = tensor
        elif key == "sink":
            self.sink_weight = tensor
        elif key == "distance_bias" and self.distance_bias is not None:
            self.bias_table = tensor
        elif key == "value_mix" and self.value_mix is not None:
            self.mix_weight = float(tensor.reshape(()).item())
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        device = self.qkv_weight.device
        if self.fixed_sink is not None:
            self.sink_weight = torch.full((self.num_heads,), self.fixed_sink, dtype=torch.float32, device=device)
        if self.distance_slope_bits is not None:
            slopes = [2.0 ** (-self.distance_slope_bits * (head + 1) / self.num_heads) for head in range(self.num_heads)]
            self.slopes = torch.tensor(slopes, dtype=torch.float64).to(torch.float32).to(device)
        if self.distance_bias is not None:
            self.bias_table = self._bias_by_distance(self.bias_table).to(device)
        # the general path adds biases in float32 behind the products, which then take the kernels for few rows
        self.conv_bias = None if self.qkv_bias is None else self.qkv_bias[:self.conv_channels].float().contiguous()
        self.o_bias_f32 = None if self.o_bias is None else self.o_bias.float().contiguous()
        if self.qkv_bias is not None and self.qkv_weight.dtype != torch.float32:
            self.qkv_bias = self.qkv_bias.to(self.qkv_weight.dtype)
        if self.o_bias is not None and self.o_weight.dtype != torch.float32:
            self.o_bias = self.o_bias.to(self.o_weight.dtype)

    def _bias_by_distance(self, table: Tensor) -> Tensor:
        """The loaded table [rows, heads] laid out by distance, float32 [heads, span]: entry n is the row of
        distance n's bucket; the last entry serves every distance from span - 1 on (with a window, no
        distance beyond window - 1 is ever read; without one, all distances from the reach on share the
        last row)."""
        import math

        rows, reach = self.distance_bias
        half = rows // 2
        last = int(math.ceil(reach)) if self.window is None else min(self.window - 1, int(math.ceil(reach)))
        buckets = []
        for n in range(last + 1):
            if n < half:
                buckets.append(n)
            else:
                buckets.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (rows - half)))))
        index = torch.tensor(buckets, dtype=torch.long, device=table.device)
        return table.to(torch.float32).index_select(0, index).t().contiguous()

    def split_qkv_weight(self) -> dict[str, Tensor]:
        """The three projection matrices back out of the fused one."""
        named = {"q": "q_proj", "k": "k_proj", "v": "v_proj"}
        return {named[key]: self.qkv_weight[start:start + size] for key, (start, size) in self._rows.items() if key in named}

    # ------------------------------------------------------------ running
    def cache_needs(self) -> CacheNeeds:
        paged = PagedKV(self.num_kv_heads, self.head_dim, self.window,
                        None if self.value_dim == self.head_dim else self.value_dim, chunk=self.chunk)
        if self.conv_taps < 2:        # one tap looks at the token's own row only: nothing to keep
            return CacheNeeds(paged=paged)
        # the last taps - 1 projected rows (q, k and v channels), exact in float32
        return CacheNeeds(paged=paged, state={self.CONV_STATE: FixedState((self.conv_taps - 1, self.conv_channels), torch.float32)})

    CONV_STATE = "conv"

    takes_stream = True

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True,
                stream: Tensor | None = None) -> Tensor | None:
        rotary = self.position.rotary()
        inv_freq, rotary_dim = rotary if rotary is not None else (None, 0)
        if self.general:
            return self._forward_general(x, batch, cache, writes_cache, stream, inv_freq, rotary_dim)
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 1.0
        if writes_cache:
            if self._single_tokens_only(batch, x, cache, rotary_dim):
                # norms, rotation, cache write and attention in one launch, which also adds up
                # the projection's partial sums where the product is faster with K in parts
                qkv = ops.linear_in_parts(x, self.qkv_weight) if self.qkv_bias is None else None
                if qkv is None:
                    qkv = ops.linear(x, self.qkv_weight, self.qkv_bias)
                attn = torch.empty((x.shape[0], self.q_size), dtype=x.dtype, device=x.device)
                ops.decode_attention_prepare(
                    qkv, self.q_norm, self.k_norm, inv_freq, cache.key_pages, cache.value_pages, attn,
                    batch.cu_q, batch.ctx_len, cache.block_table, q_heads=self.num_heads,
                    kv_heads=self.num_kv_heads, head_dim=self.head_dim, eps=eps, scale=self.scale,
                    window=self.window, max_ctx=batch.max_ctx)
                return ops.linear_update(attn, self.o_weight, self.o_bias, stream)
            qkv = ops.linear(x, self.qkv_weight, self.qkv_bias)
        else:  # another call wrote the keys and values this one reads: only q is needed
            bias = None if self.qkv_bias is None else self.qkv_bias[:self.q_size]
            qkv = ops.linear(x, self.qkv_weight[:self.q_size], bias)
        ops.qk_norm_rope_write(
            qkv, self.q_norm, self.k_norm, inv_freq, batch.positions, batch.token_seq,
            cache.block_table, cache.key_pages, cache.value_pages, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, rotary_dim=rotary_dim, eps=eps,
            write_kv=writes_cache)
        attn = torch.empty((x.shape[0], self.q_size), dtype=x.dtype, device=x.device)
        ops.paged_attention(
            qkv, cache.key_pages, cache.value_pages, attn, batch.cu_q, batch.ctx_len, cache.block_table,
            num_seqs=batch.num_seqs, max_q_len=batch.max_q_len, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
            num_decode=batch.num_decode, max_ctx=batch.max_ctx)
        return ops.linear_update(attn, self.o_weight, self.o_bias, stream)   # float32 update for the residual sum

    def _forward_general(self, x: Tensor, batch, cache: CacheView, writes_cache: bool, stream, inv_freq,
                         rotary_dim: int) -> Tensor | None:
        if writes_cache != self.own_kv or (not writes_cache and self.whole_norm_eps is None):
            raise ValueError("the general attention path writes its own keys and values, except for a layer that "
                             "has none and reads another call's")
        qkv = ops.linear(x, self.qkv_weight)        # [T, q | k | v (| gate)]; the bias is added by the kernel below
        q = torch.empty((x.shape[0], self.q_size), dtype=x.dtype, device=x.device)
        magnitude = self.position.magnitude()
        if self.whole_norm_eps is not None:
            ops.whole_norm_rope_write(
                qkv, self.q_norm, self.k_norm, inv_freq, batch.positions, batch.token_seq, cache.block_table,
                cache.key_pages, cache.value_pages, q, q_heads=self.num_heads, kv_heads=self.num_kv_heads,
                head_dim=self.head_dim, value_dim=self.value_dim, rotary_dim=rotary_dim, eps=self.whole_norm_eps,
                magnitude=magnitude, write_kv=writes_cache)
        elif magnitude != 1.0:
            raise ValueError("scaled cosines and sines come with the whole-projection norm's kernel only")
        else:
            self._conv_rope(qkv, q, batch, cache, inv_freq, rotary_dim)
        attn = torch.empty((x.shape[0], self.out_size), dtype=x.dtype, device=x.device)
        ops.masked_attention(
            q, cache.key_pages, cache.value_pages, attn, batch.cu_q, batch.ctx_len, cache.block_table,
            num_seqs=batch.num_seqs, max_q_len=batch.max_q_len, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, value_dim=self.value_dim, scale=self.scale,
            window=self.window, chunk=self.chunk, sink=self.sink_weight, slopes=self.slopes, dist_bias=self.bias_table,
            gate=qkv[:, self.conv_channels:] if self.output_gate else None, num_decode=batch.num_decode,
            max_ctx=batch.max_ctx, softcap=self.softcap, head_gate=self.head_gate)
        update = ops.linear_update(attn, self.o_weight)
        return update if self.o_bias_f32 is None else ops.add_bias(update, self.o_bias_f32)

    def _conv_rope(self, qkv: Tensor, q: Tensor, batch, cache: CacheView, inv_freq, rotary_dim: int) -> None:
        mixing = {}
        if self.value_mix == "source":
            kept = torch.empty((qkv.shape[0], self.v_size), dtype=qkv.dtype, device=qkv.device)
            batch.carry[self.value_mix_key] = kept
            mixing = {"v_keep": kept}
        elif self.value_mix == "blend":
            if self.value_mix_key not in batch.carry:
                raise ValueError(f"{self.prefix}: no earlier layer of the step left the values '{self.value_mix_key}'")
            mixing = {"v_from": batch.carry[self.value_mix_key], "v_mix": self.mix_weight}
        ops.conv_rope_norm_write(
            qkv, self.conv_bias, self.conv_weight, cache.states[self.CONV_STATE] if self.conv_taps > 1 else None, inv_freq,
            batch.positions, batch.token_seq, batch.cu_q, batch.state_slots, cache.block_table,
            cache.key_pages, cache.value_pages, q, num_seqs=batch.num_seqs, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, value_dim=self.value_dim,
            rotary_dim=rotary_dim, unit_norm_eps=self.unit_norm_eps if self.qk_norm_eps is None else self.qk_norm_eps,
            taps=self.conv_taps, norm_weight_q=self.q_norm if self.qk_norm_eps is not None else None,
            norm_weight_k=self.k_norm if self.qk_norm_eps is not None else None,
            norm_first=self.qk_norm_eps is not None, **mixing)

    def _single_tokens_only(self, batch, x: Tensor, cache: CacheView, rotary_dim: int) -> bool:
        """Every sequence of the step brings one token, and the sizes are ones that the
        decode kernel prepares queries and keys for itself."""
        return (batch.num_decode is not None and batch.num_decode == batch.num_seqs == x.shape[0]
                and ops.decode_prepare_supported(
                    x.dtype, q_heads=self.num_heads, kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                    rotary_dim=rotary_dim, block_size=cache.key_pages.shape[2]))

    def token_inputs(self):
        return self.position.token_inputs()

    def kernel_libraries(self):
        if self.general:
            return {"whole_norm_rope" if self.whole_norm_eps is not None else "conv_rope", "attention_masked", "attention_decode", "attention_prefill", "stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}
        return {"qk_rope", "attention_generic", "attention_decode", "attention_prefill", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


register_part("mixer", "gqa_attention", GroupedQueryAttention)
