"""A selective state-space mixer (Mamba): a recurrence per channel whose decay, input and read-out
depend on the token.

In order: one product gives ``[x | z]`` (each ``inner`` wide); x passes a short causal convolution
per channel with a bias and SiLU; a second product of x gives the step size's low-rank input
(``dt_rank``), B and C (``state`` wide each); ``dt = softplus(W_dt . + b_dt)``, one per channel;
``A = -exp(A_log)`` [inner, state]; per channel c and state n

    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n,      y_c = sum_n S[c, n] C_n + D_c x_c;

then ``y * silu(z)`` and the output product.  Per request the state S (float32) and the last
taps - 1 rows of x ahead of the convolution are kept in a state slot, so a request may be cut into
steps anywhere.  Step sizes, their softplus, the decays' exponentials, B, C, the state and the
read-out are float32 in both compute modes; the products, the convolution's activation and the
gate's input are in the compute dtype.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..cache.spec import CacheNeeds, CacheView, FixedState
from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, Mixer, ParamSpec


class SelectiveScanMixer(Mixer):
    DEFAULT_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
                     "a_log": "A_log", "d": "D", "o": "o"}
    STATE, CONV_STATE = "scan", "conv"

    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, inner: int, state: int, dt_rank: int,
                 conv_taps: int, names: dict[str, str] | None = None) -> None:
        super().__init__(ctx, prefix)
        if not 1 <= state <= 256:
            raise ValueError(f"between 1 and 256 states a channel, not {state}")
        if not 1 <= conv_taps <= 8:
            raise ValueError(f"a short convolution has 1 to 8 taps, not {conv_taps}")
        self.hidden_size, self.inner, self.state, self.dt_rank, self.conv_taps = hidden_size, inner, state, dt_rank, conv_taps
        self.names = dict(self.DEFAULT_NAMES, **(names or {}))
        self.tensors: dict[str, Tensor] = {}

    def shapes(self) -> dict[str, tuple[tuple[int, ...], str, str]]:
        c, n, r, w = self.inner, self.state, self.dt_rank, self.hidden_size
        return {"in": ((2 * c, w), "matrix", "normal"), "conv": ((c, self.conv_taps), "vector", "taps"),
                "conv_bias": ((c,), "vector", "small"), "x": ((r + 2 * n, c), "matrix", "unit"),
                "dt": ((c, r), "matrix", "unit"), "dt_bias": ((c,), "vector", "unit"),
                "a_log": ((c, n), "vector", "unit"), "d": ((c,), "vector", "norm"), "o": ((w, c), "matrix", "normal")}

    def param_specs(self):
        return {self.name(self.names[key]): ParamSpec(shape, kind=kind, init=init)
                for key, (shape, kind, init) in self.shapes().items()}

    def set_param(self, name: str, tensor: Tensor) -> None:
        local = name[len(self.prefix) + 1:] if self.prefix else name
        key = next((k for k, leaf in self.names.items() if leaf == local), None)
        if key is None:
            raise KeyError(name)
        self.tensors[key] = tensor

    def finalize(self) -> None:
        t = self.tensors
        # the step size's input and B | C as two products of the same activations: the first stays in the
        # compute dtype (it feeds a product), the second stores float32 (it enters the recurrence)
        t["x_dt"] = t["x"][:self.dt_rank].contiguous()
        t["x_bc"] = t["x"][self.dt_rank:].contiguous()
        del t["x"]
        t["a"] = (-torch.exp(t["a_log"].to(torch.float32))).contiguous()
        del t["a_log"]
        for key in ("conv", "conv_bias", "dt_bias", "d"):
            t[key] = t[key].to(torch.float32).contiguous()

    def cache_needs(self) -> CacheNeeds:
        states = {self.STATE: FixedState((self.inner, self.state), torch.float32)}
        if self.conv_taps > 1:
            states[self.CONV_STATE] = FixedState((self.conv_taps - 1, self.inner), torch.float32)
        return CacheNeeds(state=states)

    def forward(self, x: Tensor, batch, cache: CacheView, writes_cache: bool = True) -> Tensor:
        t = self.tensors
        xz = ops.linear(x, t["in"])                                   # [T, x | z]
        conv_state = cache.states[self.CONV_STATE] if self.conv_taps > 1 else None
        u = ops.causal_conv_act(xz[:, :self.inner], t["conv"], t["conv_bias"], conv_state, batch.token_seq, batch.cu_q,
                                batch.state_slots, num_seqs=batch.num_seqs, act="silu")
        dt_lin = ops.linear(ops.linear(u, t["x_dt"]), t["dt"], out_dtype=torch.float32)
        bc = ops.linear(u, t["x_bc"], out_dtype=torch.float32)
        y = ops.selective_scan(u, dt_lin, t["dt_bias"], t["a"], bc, t["d"], xz[:, self.inner:], cache.states[self.STATE],
                               batch.cu_q, batch.state_slots, num_seqs=batch.num_seqs)
        return ops.linear_update(y, t["o"])

    def kernel_libraries(self):
        return {"selective_scan", "conv_rope", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide"}


register_part("mixer", "selective_scan", SelectiveScanMixer)
