"""A mixture of small gated feed-forward layers chosen per token by a router.

Router: ``z = W_r x + b_r`` in float32; the ``top`` experts with the largest logits are chosen and
their weights are the softmax over the chosen logits alone.  Expert (no biases):
``g = min(W_gate x, limit)``, ``u = clamp(W_up x, -limit, limit)``,
``y = W_down (g * sigmoid(alpha g) * (u + 1))``.  The output is the weighted sum of the chosen
experts' outputs, plus a shared expert of the same form (sizes and limit of its own) that every
token takes.

Options: ``scoring`` "sigmoid" (a chosen expert's weight is the sigmoid of its own logit, not
renormalised over the chosen); ``form`` "silu" (``y = W_down (silu(W_gate x) * (W_up x))``, no
bounds); ``weight_input`` (the weight multiplies the expert's input, ``expert(w x)``, instead of
its output; since the first products are linear, they are scaled behind their sums);
``router_bias`` False (the router has no bias tensor); ``scoring`` "softmax_all" (scores are the
softmax over all experts' logits; experts are chosen by score plus a stored ``correction`` per
expert, within the ``keep_groups`` best of ``groups`` equal runs of neighbouring experts, a run
being as good as its best corrected score; a chosen expert's weight is its own score over the
sum of the chosen scores, times ``route_scale``); ``shared_gate`` (the shared expert's output times
``sigmoid(w_g . x)``, one number a token, w_g a tensor of one row; its logit is formed with the
router's, in float32).

A step sorts its (token, choice) pairs by expert on the device and runs two grouped products over
the sorted rows (gate and up with the activation as their ending, then down, weighted by the
router); nothing is decided on the host, so steps are captured like any other.  The update comes
back in parts, one per choice (the shared expert's output joins the first), which the next norm adds
up in that order: a token's sum does not depend on what else is in the step.
"""

from __future__ import annotations

import torch
from torch import Tensor

from ..kernels import ops
from ..registry import register_part
from .base import BuildContext, FeedForward, ParamSpec


class RoutedExperts(FeedForward):
    def __init__(self, ctx: BuildContext, prefix: str, *, hidden_size: int, experts: int, top: int,
                 intermediate_size: int, limit: float | None = None, alpha: float = 1.702, shared_size: int | None = None,
                 shared_limit: float | None = None, names: dict[str, str] | None = None, scoring: str = "softmax",
                 form: str = "bounded", weight_input: bool = False, router_bias: bool = True, groups: int = 1,
                 keep_groups: int = 1, route_scale: float = 1.0, shared_gate: bool = False) -> None:
        """``names``: what the tensors are called behind the prefix; ``expert`` is a pattern with
        ``{e}`` for the expert's number."""
        super().__init__(ctx, prefix)
        if not 1 <= top <= experts:
            raise ValueError(f"a token takes between one and all {experts} experts, not {top}")
        if top > 16 or experts > 1024:
            raise ValueError("up to 16 experts a token out of up to 1,024")
        self.hidden_size = hidden_size
        self.experts, self.top = experts, top
        self.intermediate_size = intermediate_size
        if scoring not in ("softmax", "sigmoid", "softmax_all") or form not in ("bounded", "silu"):
            raise ValueError(f"unknown scoring '{scoring}' or form '{form}'")
        if scoring == "softmax_all":
            if not 1 <= groups <= 64 or experts % groups or not 1 <= keep_groups <= groups or top > experts // groups * keep_groups:
                raise ValueError(f"{experts} experts do not form {groups} equal groups of which {keep_groups} hold {top} choices")
            if router_bias or weight_input:
                raise ValueError("scores over all experts come without a router bias and weigh the experts' outputs")
        elif groups != 1 or keep_groups != 1 or route_scale != 1.0:
            raise ValueError("groups and a factor on the weights come with scoring 'softmax_all'")
        if shared_gate and not shared_size:
            raise ValueError("a gate on the shared expert needs a shared expert")
        self.groups, self.keep_groups, self.route_scale, self.shared_gate = int(groups), int(keep_groups), float(route_scale), bool(shared_gate)
        if form == "bounded" and limit is None:
            raise ValueError("the bounded activation needs a limit")
        self.scoring, self.form, self.weight_input, self.has_router_bias = scoring, form, bool(weight_input), bool(router_bias)
        self.limit, self.alpha = float(limit or 0.0), float(alpha)
        self.shared_size = shared_size
        self.shared_limit = float(self.limit if shared_limit is None else shared_limit)
        self.names = dict({"expert": "experts.{e}", "shared": "shared", "router": "router.weight", "router_bias": "router.bias",
                           "gate": "gate", "up": "up", "down": "down", "correction": "correction", "shared_gate": "shared.gate_proj"},
                          **(names or {}))
        self.correction: Tensor | None = None
        self.router_rows: Tensor | None = None      # with a gate on the shared expert: the router's rows, then the gate's row
        self.router_weight: Tensor | None = None
        self.router_bias: Tensor | None = None
        self.gate_up: Tensor | None = None          # [experts, 2 F, H]: an expert's gate rows, then its up rows
        self.down: Tensor | None = None             # [experts, H, F]
        self.shared_gate_up: Tensor | None = None   # [2 Fs, H]
        self.shared_down: Tensor | None = None

    def _expert_name(self, expert: int | None, which: str) -> str:
        owner = self.names["shared"] if expert is None else self.names["expert"].format(e=expert)
        return self.name(f"{owner}.{self.names[which]}")

    def param_specs(self):
        f, h = self.intermediate_size, self.hidden_size
        specs = {self.name(self.names["router"]): ParamSpec((self.experts, h), init="router")}
        if self.scoring == "softmax_all":     # a checkpoint without it: no correction
            specs[self.name(self.names["correction"])] = ParamSpec((self.experts,), kind="vector", init="small", optional=True)
        if self.shared_gate:
            specs[self.name(self.names["shared_gate"])] = ParamSpec((1, h), init="router")
        if self.has_router_bias:
            specs[self.name(self.names["router_bias"])] = ParamSpec((self.experts,), kind="vector", init="small")
        for expert in range(self.experts):
            specs[self._expert_name(expert, "gate")] = ParamSpec((f, h))
            specs[self._expert_name(expert, "up")] = ParamSpec((f, h))
            specs[self._expert_name(expert, "down")] = ParamSpec((h, f))
        if self.shared_size:
            specs[self._expert_name(None, "gate")] = ParamSpec((self.shared_size, h))
            specs[self._expert_name(None, "up")] = ParamSpec((self.shared_size, h))
            specs[self._expert_name(None, "down")] = ParamSpec((h, self.shared_size))
        self._owners = {}
        for expert in [*range(self.experts), None] if self.shared_size else range(self.experts):
            for which in ("gate", "up", "down"):
                self._owners[self._expert_name(expert, which)] = (expert, which)
        return specs

    def set_param(self, name: str, tensor: Tensor) -> None:
        f, h = self.intermediate_size, self.hidden_size
        if name == self.name(self.names["router"]) or (self.shared_gate and name == self.name(self.names["shared_gate"])):
            if not self.shared_gate:
                self.router_weight = tensor.contiguous()
                return
            if self.router_rows is None:
                self.router_rows = torch.empty((self.experts + 1, h), dtype=tensor.dtype, device=tensor.device)
                self.router_weight = self.router_rows[:self.experts]
            if tensor.dtype != self.router_rows.dtype:
                raise ValueError(f"{name}: the router and the shared expert's gate must be stored in one dtype")
            if name == self.name(self.names["router"]):
                self.router_rows[:self.experts].copy_(tensor)
            else:
                self.router_rows[self.experts:].copy_(tensor)
            return
        if self.scoring == "softmax_all" and name == self.name(self.names["correction"]):
            self.correction = tensor.contiguous()
            return
        if self.has_router_bias and name == self.name(self.names["router_bias"]):
            self.router_bias = tensor.contiguous()
            return
        if not hasattr(self, "_owners"):
            self.param_specs()
        if name not in self._owners:
            raise KeyError(name)
        expert, which = self._owners[name]
        if expert is None:
            if which == "down":
                self.shared_down = tensor
                return
            if self.shared_gate_up is None:
                self.shared_gate_up = torch.empty((2 * self.shared_size, h), dtype=tensor.dtype, device=tensor.device)
            start = 0 if which == "gate" else self.shared_size
            self.shared_gate_up[start:start + self.shared_size].copy_(tensor)
            return
        if which == "down":
            if self.down is None:
                self.down = torch.empty((self.experts, h, f), dtype=tensor.dtype, device=tensor.device)
            self.down[expert].copy_(tensor)
            return
        if self.gate_up is None:
            self.gate_up = torch.empty((self.experts, 2 * f, h), dtype=tensor.dtype, device=tensor.device)
        start = 0 if which == "gate" else f
        self.gate_up[expert, start:start + f].copy_(tensor)

    def finalize(self) -> None:
        if self.gate_up.dtype != self.down.dtype or self.gate_up.dtype != self.router_weight.dtype:
            raise ValueError(f"{self.prefix}: the experts' matrices and the router must be stored in one dtype")

    def forward(self, x: Tensor, batch=None) -> Tensor:
        tokens = x.shape[0]
        gate_logits, gate_column = None, 0
        if self.scoring == "softmax_all":
            chosen, weights, logits = ops.moe_route_grouped(
                x, self.router_rows if self.shared_gate else self.router_weight, self.correction, experts=self.experts,
                top=self.top, groups=self.groups, keep=self.keep_groups, scale=self.route_scale)
            gate_logits, gate_column = logits, self.experts
        else:
            chosen, weights = ops.moe_route(x, self.router_weight, self.router_bias, self.top, self.scoring)
            if self.shared_gate:
                gate_logits = ops.linear(x, self.router_rows[self.experts:], out_dtype=torch.float32)
        shared = None
        if self.shared_size:
            if self.form == "silu":     # the gated SiLU of the dense feed-forward, with its fused kernels
                act = ops.linear_swiglu(x, self.shared_gate_up)
            else:
                act = ops.linear_gated(x, self.shared_gate_up, limit=self.shared_limit, alpha=self.alpha)
            shared = ops.linear_update(act, self.shared_down)
            if self.shared_gate:
                ops.gate_rows(shared, gate_logits, gate_column)
        update = torch.empty((self.top, tokens, self.hidden_size), dtype=torch.float32, device=x.device)
        return ops.moe_experts(x, chosen, weights, self.gate_up, self.down, update, limit=self.limit, alpha=self.alpha,
                               extra=shared, form=self.form, weight_input=self.weight_input)

    def kernel_libraries(self):
        return {"moe", "rowwise", "stream_ops", "gemm_f32", "gemm_skinny", "gemm_mid", "gemm_wide", "gemm_tile"}


register_part("feed_forward", "routed_experts", RoutedExperts)
