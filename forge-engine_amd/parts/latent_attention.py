"""Causal attention whose keys and values are made from one small cached vector per token.

With x the mixer's input, H heads, per head ``head_dim`` plain and ``rot_dim`` rotated query/key
dims and ``value_dim`` value dims:

* queries through a bottleneck: ``a = rmsnorm(W_dq x)`` (weighted, ``q_rank`` wide), ``q = W_uq a``,
  laid out head by head as [plain | rotated];
* what a token leaves in the cache: ``c = rmsnorm(first kv_rank rows of W_dkv x)`` (weighted) and
  ``r = rotate(last rot_dim rows of W_dkv x)``, one key part shared by all heads;
* head h's key of token j is ``[W_uk[h] c_j | r_j]`` and its value ``W_uv[h] c_j``; scores are
  ``(q_plain . W_uk[h] c_j + q_rot . r_j) * scale``, softmax over j <= i, output ``W_o`` on the
  concatenated heads.

Keys and values are never made.  ``q_plain . W_uk[h] c = (W_uk[h]^T q_plain) . c``, so every head's
query is taken through its key up-projection once and attention then runs over the cached rows
``[c | r]`` themselves, all heads sharing them like the query heads of one key/value head; the values
are the first ``kv_rank`` dims of those rows, and ``W_uv[h]`` is applied once to the attention's
result.  The cache holds one row ``[c | r]`` a token as its key pages and ``c`` a second time in
transposed value pages (the layout the matrix-core kernel reads its second operand in):
``2 kv_rank + rot_dim`` numbers a token, whatever the number of heads.

A layer with ``own_kv`` False has no ``W_dkv``: it is scheduled to read the pages of an earlier layer
of the same geometry, with its own queries, ``W_uk``, ``W_uv`` and ``W_o``.

The rotation is the position part's (rotate-half pairing over its first ``rotary_dim`` dims, of the
``rot_dim`` wide part).  Norms, angles, scores and softmax are float32; the down-projections are
stored float32 for the norms.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, PagedKV
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec, build_part
from .plan import PartSpec


class LatentAttention(Mixer):
    DEFAULT_NAMES = {"dq": "q_down.weight", "dq_norm": "q_down.norm", "uq": "q_up.weight", "dkv": "kv_down.weight",
                     "dkv_norm": "kv_down.norm", "uk": "k_up.weight", "uv": "v_up.weight", "o": "o_proj.weight"}

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int,
                 value_dim: int, q_rank: int, kv_rank: int, eps: float, position: PartSpec, scale: float | None = None,
                 own_kv: bool = True, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix)
        if min(num_heads, head_dim, value_dim, q_rank, kv_rank) < 1 or rot_dim < 0:
            raise ValueError("heads, head sizes and ranks must be positive")
        if kv_rank + rot_dim > ops.MASKED_MAX_KEY_DIM or kv_rank > ops.MASKED_MAX_VALUE_DIM:
            raise ValueError(f"cached rows of up to {ops.MASKED_MAX_KEY_DIM} numbers with a latent of up to "
                             f"{ops.MASKED_MAX_VALUE_DIM}, not {kv_rank} + {rot_dim}")
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.head_dim, self.rot_dim, self.value_dim = head_dim, rot_dim, value_dim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.row_dim = kv_rank + rot_dim                 # what a token leaves in the cache
        self.q_head = head_dim + rot_dim
        self.eps = float(eps)
        self.scale = (head_dim + rot_dim) ** -0.5 if scale is None else float(scale)
        self.own_kv = own_kv
        self.names = dict(self.DEFAULT_NAMES, **(names or {}))
        self.position = build_part("position", position, ctx)
        rotary = self.position.rotary()
        if rotary is not None and rotary[1] > rot_dim:
            raise ValueError(f"{rotary[1]} rotated dims do not fit a rotated part of {rot_dim}")
        if self.position.magnitude() != 1.0:
            raise ValueError("attention through a latent takes a plain rotation")
        self.down_rows = q_rank + (self.row_dim if own_kv else 0)
        self.down_weight: Tensor | None = None      # [q_rank (+ kv_rank + rot_dim), hidden]: one product for both bottlenecks
        self.q_norm: Tensor | None = None
        self.kv_norm: Tensor | None = None
        self.uq_weight: Tensor | None = None
        self.uk: Tensor | None = None               # [heads, head_dim, kv_rank]
        self.uv_t: Tensor | None = None             # [heads, kv_rank, value_dim]
        self.o_weight: Tensor | None = None

    def param_specs(self):
        n = {key: self.name(leaf) for key, leaf in self.names.items()}
        heads, hidden = self.num_heads, self.hidden_size
        specs = {
            n["dq"]: ParamSpec((self.q_rank, hidden)),
            n["dq_norm"]: ParamSpec((self.q_rank,), kind="vector", init="norm"),
            n["uq"]: ParamSpec((heads * self.q_head, self.q_rank)),
            n["uk"]: ParamSpec((heads * self.head_dim, self.kv_rank)),
            n["uv"]: ParamSpec((heads * self.value_dim, self.kv_rank)),
            n["o"]: ParamSpec((hidden, heads * self.value_dim)),
        }
        if self.own_kv:
            specs[n["dkv"]] = ParamSpec((self.row_dim, hidden))
            specs[n["dkv_norm"]] = ParamSpec((self.kv_rank,), kind="vector", init="norm")
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        local = name[len(self.prefix) + 1:] if self.prefix else name
        key = next((k for k, leaf in self.names.items() if leaf == local), None)
        if key in ("dq", "dkv") and (key == "dq" or self.own_kv):
            if self.down_weight is None:
                self.down_weight = torch.empty((self.down_rows, self.hidden_size), dtype=tensor.dtype, device=tensor.device)
            if tensor.dtype != self.down_weight.dtype:
                raise ValueError(f"{name}: the down-projections of one input must be stored in one dtype")
            start = 0 if key == "dq" else self.q_rank
            self.down_weight[start:start + tensor.shape[0]].copy_(tensor)
        elif key == "dq_norm":
            self.q_norm = tensor
        elif key == "dkv_norm" and self.own_kv:
            self.kv_norm = tensor
        elif key == "uq":
            self.uq_weight = tensor
        elif key == "uk":
            self.uk = tensor.view(self.num_heads, self.head_dim, self.kv_rank)
        elif key == "uv":
            self.uv_t = tensor.view(self.num_heads, self.value_dim, self.kv_rank).transpose(1, 2).contiguous()
        elif key == "o":
            self.o_weight = tensor
        else:
            raise KeyError(name)

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(paged=PagedKV(1, self.row_dim, None, self.kv_rank))

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True) -> Tensor:
        if writes_cache != self.own_kv:
            raise ValueError(f"{self.prefix}: a layer with a down-projection of its own writes its cache, one without reads another's")
        tokens, heads = x.shape[0], self.num_heads
        rotary = self.position.rotary()
        inv_freq, rotary_dim = rotary if rotary is not None else (None, 0)
        down = ops.linear(x, self.down_weight, out_dtype=torch.float32)
        latent_q = torch.empty((tokens, self.q_rank), dtype=x.dtype, device=x.device)
        ops.latent_norm_rope_write(down, self.q_norm, self.kv_norm, inv_freq, batch.positions, batch.token_seq,
                                   cache.block_table, cache.key_pages, cache.value_pages, latent_q, q_rank=self.q_rank, kv_rank=self.kv_rank,
                                   rot_dim=self.rot_dim, rotary_dim=rotary_dim, eps=self.eps, write_kv=writes_cache)
        q = ops.linear(latent_q, self.uq_weight)                                       # [T, H * (plain | rotated)]
        through_keys = ops.heads_product(q.view(tokens, heads, self.q_head)[:, :, :self.head_dim], self.uk)    # [H, T, kv_rank]
        rows = torch.empty((tokens, heads, self.row_dim), dtype=x.dtype, device=x.device)
        ops.latent_query_pack(q, through_keys, inv_freq, batch.positions, rows, heads=heads, dim=self.head_dim,
                              rot_dim=self.rot_dim, rotary_dim=rotary_dim, kv_rank=self.kv_rank)
        read = torch.empty((tokens, heads * self.kv_rank), dtype=x.dtype, device=x.device)
        ops.latent_attention(rows.view(tokens, heads * self.row_dim), cache.key_pages, cache.value_pages, read, batch.cu_q, batch.ctx_len,
                             cache.block_table, num_seqs=batch.num_seqs, max_q_len=batch.max_q_len, heads=heads,
                             row_dim=self.row_dim, value_dim=self.kv_rank, scale=self.scale, num_decode=batch.num_decode,
                             max_ctx=batch.max_ctx)
        values = ops.heads_product(read.view(tokens, heads, self.kv_rank), self.uv_t)  # [H, T, value_dim]
        attn = values.transpose(0, 1).reshape(tokens, heads * self.value_dim)
        return ops.linear_update(attn, self.o_weight)

    def token_inputs(self):
        return self.position.token_inputs()

    def kernel_libraries(self):
        return {"latent", "attention_latent", "attention_masked", "stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


register_part("mixer", "latent_attention", LatentAttention)
