"""Mufenex as data: its config.json typed, and turned into a `ModelSpec`.

A decoder-only model whose layers are listed one by one in config.json (`layers`: each entry a
`type`, the mixer's sizes under `mixer`, and `mlp` or null), so two layers of one model may differ in
every size.  What the design fixes is written here; what config.json gives is read from there:

  embedding   x = embed[token] * embedding.scale + sinusoidal position vector (base 10000 over
              the model's width, sin at even entries, cos at odd ones)
  layer       x <- x + norm1(mixer(x)); x <- x + norm2(ff(x)) (block "branchnorm": the sublayers read the
              stream itself, RMSNorm with norm.eps on their output); `mlp: null` leaves the second out
  attention   grouped-query attention with value heads of their own size (`vdim`), RMSNorm over the
              whole q and the whole k projection, no rotation; score = (q . k) * scale, soft-capped
              (softcap * tanh(score / softcap)), minus slope_h * (i - j) with slope_h = 2^(-8 (h + 1) / H);
              a sliding window of mask.size keys; in the layers that say `v_mix`, but the first of
              them, the values are blended with the first such layer's values of the same token by the
              layer's scalar `vmix`, and the blended values are what the cache keeps
  mlp         dense: down(gelu_tanh(gate x) * (up x)); moe: a router with a bias chooses `top` of
              `experts` gated silu experts, weighted by the softmax over the chosen logits
  output      RMSNorm `final.norm`, `head`, logits soft-capped by logit_softcap

Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.{q,k,v,o,q.norm,k.norm,vmix}`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,router.b,e<j>.gate,e<j>.up,e<j>.down}`, `final.norm`, `head`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.model_config import ConfigError, _require, _typed
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import ModelFamily, register_architecture

SINUSOID_BASE = 10000.0           # of the position vector
SLOPE_EXPONENT = 8.0              # slope of head h of H: 2^(-SLOPE_EXPONENT (h + 1) / H)
DEFAULT_POSITIONS = 1 << 16       # config.json names no longest sequence: what the engine plans its tables for


def _opt(raw: Dict[str, Any], key: str, typ, where: str):
    return None if raw.get(key) is None else _typed(raw[key], key, typ, where)


@dataclass(frozen=True)
class MufenexMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    window: Optional[int] = None          # mask.size
    v_mix: bool = False

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "MufenexMixer":
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: 'mixer' must be an object")
        mask = raw.get("mask")
        if mask is not None and not isinstance(mask, dict):
            raise ConfigError(f"{where}: 'mask' must be an object or null")
        dim = _require(raw, "dim", int, where)
        m = cls(heads=_require(raw, "heads", int, where), kv_heads=_require(raw, "kv_heads", int, where), dim=dim,
                vdim=_opt(raw, "vdim", int, where) or dim,
                scale=_opt(raw, "scale", float, where) if raw.get("scale") is not None else float(dim) ** -0.5,
                softcap=_opt(raw, "softcap", float, where),
                window=_opt(mask, "size", int, where) if mask else None,
                v_mix=bool(_opt(raw, "v_mix", bool, where)))
        if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
            raise ConfigError(f"{where}: {m.heads} heads of size {m.dim}/{m.vdim} on {m.kv_heads} kv heads cannot be run")
        if m.softcap is not None and not m.softcap > 0:
            raise ConfigError(f"{where}: softcap must be positive or absent")
        if m.window is not None and m.window <= 0:
            raise ConfigError(f"{where}: mask.size must be positive or absent")
        return m

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim,
                               "scale": self.scale, "v_mix": self.v_mix}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class MufenexMlp:
    kind: str                     # "dense" or "moe"
    ff: int                       # dense: the hidden size; moe: one expert's
    experts: int = 0
    top: int = 0

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> Optional["MufenexMlp"]:
        if raw is None:
            return None
        if not isinstance(raw, dict):
            raise ConfigError(f"{where}: 'mlp' must be an object or null")
        kind = _require(raw, "kind", str, where)
        if kind == "dense":
            m = cls("dense", _require(raw, "ff", int, where))
        elif kind == "moe":
            expert, router = raw.get("expert"), raw.get("router")
            if not isinstance(expert, dict) or not isinstance(router, dict):
                raise ConfigError(f"{where}: a moe mlp needs 'expert' and 'router' objects")
            m = cls("moe", _require(expert, "ff", int, where), _require(router, "experts", int, where),
                    _require(router, "top", int, where))
            if not (0 < m.top <= m.experts):
                raise ConfigError(f"{where}: {m.top} of {m.experts} experts cannot be chosen")
        else:
            raise ConfigError(f"{where}: unknown mlp kind {kind!r} (dense, moe)")
        if m.ff <= 0:
            raise ConfigError(f"{where}: ff must be positive")
        return m

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class MufenexLayer:
    type: str
    mixer: MufenexMixer
    mlp: Optional[MufenexMlp]


@dataclass(frozen=True)
class MufenexConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[MufenexLayer, ...]
    logit_softcap: Optional[float] = None
    max_positions: int = DEFAULT_POSITIONS
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Mufenex"

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "MufenexConfig":
        emb, norm, layers = raw.get("embedding") or {}, raw.get("norm") or {}, raw.get("layers")
        if not isinstance(layers, list):
            raise ConfigError(f"{where}: 'layers' must be a list")
        out = []
        for i, l in enumerate(layers):
            at = f"{where}: layers[{i}]"
            if not isinstance(l, dict):
                raise ConfigError(f"{at} must be an object")
            kind = _require(l, "type", str, at)
            if kind != "attention":
                raise ConfigError(f"{at}: unknown layer type {kind!r} (attention)")
            out.append(MufenexLayer(kind, MufenexMixer.from_dict(l.get("mixer"), at), MufenexMlp.from_dict(l.get("mlp"), at)))
        eos = raw.get("eos_token_id")
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  embedding_scale=_opt(emb, "scale", float, where) if emb.get("scale") is not None else 1.0,
                  norm_eps=_require(norm, "eps", float, where), layers=tuple(out),
                  logit_softcap=_opt(raw, "logit_softcap", float, where),
                  max_positions=_opt(raw, "max_positions", int, where) or DEFAULT_POSITIONS,
                  eos_token_id=None if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Mufenex"])[0]))
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_positions <= 0:
            raise ConfigError(f"{where}: vocab, width and max_positions must be positive")
        if cfg.logit_softcap is not None and not cfg.logit_softcap > 0:
            raise ConfigError(f"{where}: logit_softcap must be positive or absent")
        first = cfg.first_mixed_layer()
        for i, l in enumerate(cfg.layers):
            if l.mixer.v_mix and first is not None and i != first:
                a, b = cfg.layers[first].mixer, l.mixer
                if a.kv_heads * a.vdim != b.kv_heads * b.vdim:
                    raise ConfigError(f"{where}: layers {first} and {i} blend values of different sizes")
        return cfg

    def first_mixed_layer(self) -> Optional[int]:
        """The layer whose values the other `v_mix` layers blend in: the first that says `v_mix`."""
        for i, l in enumerate(self.layers):
            if l.mixer.v_mix:
                return i
        return None

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers]}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.max_positions != DEFAULT_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


def head_slopes(heads: int) -> Tuple[float, ...]:
    """The distance bias's slope of every query head: 2^(-8 (h + 1) / H)."""
    return tuple(2.0 ** (-SLOPE_EXPONENT * (h + 1) / heads) for h in range(heads))


def mufenex_spec(cfg: MufenexConfig) -> ModelSpec:
    first = cfg.first_mixed_layer()
    layers = []
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        params: Dict[str, Any] = dict(
            hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
            bias=False, qk_norm="row", qk_norm_eps=cfg.norm_eps, window=m.window, position=None, scale=m.scale,
            score_softcap=m.softcap, distance_slopes=head_slopes(m.heads),
            names={"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "value_mix": "vmix"})
        if m.v_mix:
            params["value_mix"] = {"key": "first", "source": i == first}
        mixer = PartSpec("attention", params)
        if l.mlp is None:
            ffn = None
        elif l.mlp.kind == "dense":
            ffn = PartSpec("gated_mlp", dict(hidden_size=cfg.width, intermediate_size=l.mlp.ff, activation="gelu_tanh",
                                             names={"gate": "gate", "up": "up", "down": "down"}))
        else:
            ffn = PartSpec("routed_experts", dict(
                hidden_size=cfg.width, intermediate_size=l.mlp.ff, num_experts=l.mlp.experts, top=l.mlp.top,
                router_bias=True, activation="silu",
                names={"router": "router", "router_bias": "router.b", "gate": "e{i}.gate", "up": "e{i}.up", "down": "e{i}.down"}))
        norms = {"norm1": PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm1"))}
        if ffn is not None:
            norms["norm2"] = PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm2"))
        layers.append(LayerSpec(prefix=f"l{i}", block="branchnorm", mixer=mixer, feed_forward=ffn, norms=norms,
                                mixer_name="mix", feed_forward_name="mlp"))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", dict(name="embed", vocab_size=cfg.vocab, dim=cfg.width, scale=cfg.embedding_scale,
                                             sinusoid_base=SINUSOID_BASE)),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name="final.norm")),
        head=PartSpec("lm_head", dict(name="head", tied=False, vocab_size=cfg.vocab, dim=cfg.width,
                                      softcap=cfg.logit_softcap)),
        eos_token_ids=tuple(cfg.eos_token_id or ()))


MUFENEX = ModelFamily("mufenex", MufenexConfig, mufenex_spec)
register_architecture("Mufenex", MUFENEX)
