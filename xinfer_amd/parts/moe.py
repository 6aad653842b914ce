"""Routed experts (mixture of experts) as a feed-forward.

z = W_router x (+ b) in float32; each token takes the `top` experts with the largest z, weighted by
the softmax over the chosen logits only; an expert is a gated feed-forward without biases,
down(act(gate x) * (up x)); the result is the weighted sum of the chosen experts' outputs, in
float32.  The experts' weights are stacked at load: gate and up [E, 2F, H] (gate rows first), down
[E, H, F].  In steps of single tokens nothing is read on the host: the router's choice stays on the
device and the experts' kernels find their rows from it, so decode steps can be recorded.

Tensor names under the part's prefix (`names` of the spec replaces any of them): `router`,
`router_bias`, and per expert i `expert{i}.gate`, `expert{i}.up`, `expert{i}.down`, in which "{i}" is
the expert's number.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import FeedForward, StepContext, register_feed_forward


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True
    LIBRARY = True       # False: the hand-written kernels for every step
    NAMES = {"router": "router.weight", "router_bias": "router.bias", "gate": "experts.{i}.gate_proj.weight",
             "up": "experts.{i}.up_proj.weight", "down": "experts.{i}.down_proj.weight"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])          # of one expert
        self.experts = int(spec["num_experts"])
        self.top = int(spec["top"])
        self.router_bias = bool(spec.get("router_bias", False))
        self.activation = str(spec.get("activation", "silu"))
        if self.activation not in kernels.ACTIVATIONS:
            raise NotImplementedError(f"activation {self.activation!r} is not built ({', '.join(kernels.ACTIVATIONS)})")
        if not (0 < self.top <= self.experts):
            raise ValueError(f"{self.top} of {self.experts} experts cannot be chosen")
        self.router_w: Optional[torch.Tensor] = None     # float32 [E, H]
        self.router_b: Optional[torch.Tensor] = None     # float32 [E]
        self.gate_up: Optional[torch.Tensor] = None      # [E, 2F, H]
        self.down: Optional[torch.Tensor] = None         # [E, H, F]

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str):
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, f, e = int(spec["hidden_size"]), int(spec["intermediate_size"]), int(spec["num_experts"])
        n = cls._names(spec, prefix)
        out = [TensorDecl(n["router"], (e, h))]
        if spec.get("router_bias", False):
            out.append(TensorDecl(n["router_bias"], (e,)))
        for i in range(e):
            out += [TensorDecl(n["gate"].replace("{i}", str(i)), (f, h)), TensorDecl(n["up"].replace("{i}", str(i)), (f, h)),
                    TensorDecl(n["down"].replace("{i}", str(i)), (h, f))]
        return out

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._names(self.spec, prefix)
        self.router_w = store.get(n["router"], torch.float32, device).contiguous()
        if self.router_bias:
            self.router_b = store.get(n["router_bias"], torch.float32, device).contiguous()
        gu, dn = [], []
        for i in range(self.experts):
            g, u, d = (store.get(n[k].replace("{i}", str(i)), self.dtype, device) for k in ("gate", "up", "down"))
            gu.append(torch.cat([g, u], dim=0))
            dn.append(d)
        self.gate_up = torch.stack(gu).contiguous()
        self.down = torch.stack(dn).contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        idx, wt = kernels.moe_route(x, self.router_w, self.router_b, self.top)
        # a step that brings portions is never recorded: with many rows an expert it may read the experts' row
        # counts on the host and hand each expert's rows to the vendor library, as the dense products of many rows go
        if (ctx.max_q_len > 1 and x.dtype == torch.bfloat16 and self.LIBRARY
                and x.shape[0] * self.top >= kernels.MOE_LIBRARY_ROWS * self.experts):
            return kernels.moe_experts_library(x, self.gate_up, self.down, idx, wt, self.activation)
        return kernels.moe_experts(x, self.gate_up, self.down, idx, wt, self.activation)
