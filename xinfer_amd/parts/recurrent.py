"""Linear attention with a decaying state, as mixers: "gated_linear_attention" and "retention".

Both keep, per request and head, a float32 matrix S [key_dim, value_dim] in the request's state slot
(no pages: the cache of such a layer does not grow with the context) and do, token by token,

    S <- diag(a_t) S + k_t v_t^T        o_t = S^T q_t

then norm each head's o by its root mean square over value_dim (eps inside the root), multiply by
silu(g) with g a projection of the input of its own, and project the concatenated heads (`o`).  A state
slot holds zeros when a request runs its first token (the runner clears it), and a step leaves the state
after its last token there, so a prompt may be cut anywhere.

  gated_linear_attention   a_t = sigmoid(z_t)^(1 / tau) per key channel, z_t = A2 (A1 h) + b (a low-rank
                           projection, its rank read from A1's shape); q is multiplied by `q_scale`
                           (key_dim^-1/2 unless given); the heads' norm has a weight [value_dim] shared
                           by the heads.
  retention                a_t = decay[h], one constant a head; k is multiplied by `k_scale`
                           (key_dim^-1/2 unless given); the heads' norm has no weight.

Decays, their logarithms and exponentials, the state, o and its norm are float32 in both precisions; the
projections and the gate's activation run in the activation dtype.  q, k, v and g are one packed
product.  Tensor names under the part's prefix: q, k, v, g, o (and a1, a2, a2.b, norm); the spec's `names`
replaces any of them.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import kernels
from ..config.spec import PartSpec
from ..weights.store import TensorDecl, WeightStore
from .base import LayerCache, Mixer, StateNeed, StepContext, register_mixer
from .linear import Linear


class _DecayingState(Mixer):
    graph_safe = True
    NAMES: Dict[str, str] = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.dk = int(spec["key_dim"])
        self.dv = int(spec["value_dim"])
        self.eps = float(spec["norm_eps"])
        if min(self.hidden, self.heads, self.dk, self.dv) <= 0:
            raise ValueError(f"{self.heads} heads of {self.dk} by {self.dv} on a width of {self.hidden} cannot be run")
        self.proj: Optional[Linear] = None           # [q | k | v | g] rows
        self.o: Optional[Linear] = None

    @classmethod
    def _names(cls, spec: PartSpec, prefix: str) -> Dict[str, str]:
        given = spec.get("names") or {}
        return {k: f"{prefix}.{given.get(k, v)}" for k, v in cls.NAMES.items()}

    @classmethod
    def _declare_common(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, H, dk, dv = (int(spec[k]) for k in ("hidden_size", "num_heads", "key_dim", "value_dim"))
        n = cls._names(spec, prefix)
        return [TensorDecl(n["q"], (H * dk, h)), TensorDecl(n["k"], (H * dk, h)), TensorDecl(n["v"], (H * dv, h)),
                TensorDecl(n["g"], (H * dv, h)), TensorDecl(n["o"], (h, H * dv))]

    def _lin(self, store: WeightStore, name: str, device) -> torch.Tensor:
        t = store.get(name, None, device)
        return t.to(self.dtype) if (self.dtype == torch.float32 or t.dtype != torch.float32) else t

    def _load_common(self, store: WeightStore, prefix: str, device) -> Dict[str, str]:
        n = self._names(self.spec, prefix)
        parts = [self._lin(store, n[k], device) for k in ("q", "k", "v", "g")]
        common = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        self.proj = Linear(torch.cat([p.to(common) for p in parts], dim=0))
        self.o = Linear(self._lin(store, n["o"], device))
        return n

    def state_need(self) -> StateNeed:
        return StateNeed((self.heads, self.dk, self.dv), torch.float32)

    def _split(self, p: torch.Tensor):
        a, b = self.heads * self.dk, self.heads * self.dv
        return p[:, :a], p[:, a:2 * a], p[:, 2 * a:2 * a + b], p[:, 2 * a + b:2 * a + 2 * b]

    @staticmethod
    def _cutting(ctx: StepContext):
        """What the state's kernel may know of the step on the host: nothing in a step of single tokens (which may be
        recorded), the portions' lengths otherwise (long portions are then walked chunk by chunk, side by side)."""
        if ctx.max_q_len <= 1 or not ctx.cu_q_host:
            return {}
        cu = ctx.cu_q_host
        return dict(q_lens=[cu[b + 1] - cu[b] for b in range(ctx.num_seqs)], plan_cache=ctx.scratch)

    @staticmethod
    def _state(cache: LayerCache) -> torch.Tensor:
        if cache.state is None:
            raise RuntimeError("a mixer with a decaying state was given no state slots")
        return cache.state


@register_mixer("gated_linear_attention")
class GatedLinearAttention(_DecayingState):
    NAMES = {**_DecayingState.NAMES, "a1": "a1", "a2": "a2", "a2_bias": "a2.b", "norm": "norm"}

    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.tau = float(spec["tau"])
        self.rank = int(spec["decay_rank"])
        self.q_scale = float(spec.get("q_scale") or self.dk ** -0.5)
        if not self.tau > 0 or self.rank <= 0:
            raise ValueError(f"tau {self.tau} and the decay's rank {self.rank} must be positive")
        self.a1: Optional[Linear] = None
        self.a2: Optional[Linear] = None
        self.a2_bias = self.norm_w = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        h, H, dk, dv, r = (int(spec[k]) for k in ("hidden_size", "num_heads", "key_dim", "value_dim", "decay_rank"))
        n = cls._names(spec, prefix)
        return cls._declare_common(spec, prefix) + [
            TensorDecl(n["a1"], (r, h)), TensorDecl(n["a2"], (H * dk, r)), TensorDecl(n["a2_bias"], (H * dk,)),
            TensorDecl(n["norm"], (dv,), "norm")]

    def load(self, store: WeightStore, prefix: str, device) -> None:
        n = self._load_common(store, prefix, device)
        self.a1 = Linear(self._lin(store, n["a1"], device))
        self.a2 = Linear(self._lin(store, n["a2"], device))
        self.a2_bias = store.get(n["a2_bias"], torch.float32, device).contiguous()
        self.norm_w = store.get(n["norm"], torch.float32, device).contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        p = self.proj(x, out_dtype=self.dtype)
        q, k, v, g = self._split(p)
        # the decay's logits leave the second product in float32; their bias is added where they are read
        z = self.a2(self.a1(x, out_dtype=self.dtype), out_dtype=torch.float32)
        o = kernels.linear_scan(q, k, v, self._state(cache), ctx.state_slots, ctx.cu_q, self.heads, self.dk, self.dv,
                                z=z, z_bias=self.a2_bias, tau=self.tau, q_scale=self.q_scale, **self._cutting(ctx))
        return self.o(kernels.head_norm_gate(o, self.norm_w, self.eps, g, self.dtype), out_dtype=self.dtype)


@register_mixer("retention")
class Retention(_DecayingState):
    def __init__(self, spec: PartSpec, dtype: torch.dtype):
        super().__init__(spec, dtype)
        self.decay_values = tuple(float(d) for d in spec["decay"])
        self.k_scale = float(spec.get("k_scale") or self.dk ** -0.5)
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        self.decay: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorDecl]:
        return cls._declare_common(spec, prefix)

    def load(self, store: WeightStore, prefix: str, device) -> None:
        self._load_common(store, prefix, device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        p = self.proj(x, out_dtype=self.dtype)
        q, k, v, g = self._split(p)
        o = kernels.linear_scan(q, k, v, self._state(cache), ctx.state_slots, ctx.cu_q, self.heads, self.dk, self.dv,
                                head_decay=self.decay, k_scale=self.k_scale, **self._cutting(ctx))
        return self.o(kernels.head_norm_gate(o, None, self.eps, g, self.dtype), out_dtype=self.dtype)
