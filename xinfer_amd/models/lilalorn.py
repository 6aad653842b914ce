"""Lilalorn as data: its config.json typed, and turned into a `ModelSpec`.

A decoder-only model whose layers are listed one by one in config.json (`layers`: each entry a `type`, the
mixer's sizes under `mixer`, `mlp` or null, and optionally `weights_of`).  What the design fixes is written
here; what config.json gives is read from there:

  embedding   x = embed[token]
  layer       pre-norm with a factor m = residual_mult on both branches: x <- x + m mixer(norm1(x)), then
              x <- x + m ff(norm2(x)) (block "prenorm" with `residual_scale`); `mlp: null` leaves the second
              out.  A layer with `weights_of: j` has no tensors: it runs with layer j's, on a cache and
              state of its own (a schedule entry with a `cache_id`).
  type "gla"  gated linear attention: per head a float32 state S [dim, vdim], S <- diag(a) S + k v^T,
              o = S^T q with q scaled by dim^-1/2 and a = sigmoid(A2 (A1 h) + b)^(1 / tau) per key channel;
              o normed head by head (RMS, weight `norm` of vdim shared by the heads), times silu(g h), then `o`
  type "parallel"  two mixers on the same input, left_scale * left + right_scale * right:
              left   grouped-query softmax attention over all earlier tokens, value heads of their own
                     size, score = (q . k) * scale, rotary positions on the first rot.dims dims of q and
                     k (pairs (i, i + dims / 2), base rot.base, the frequencies stretched band by band by
                     rot.scaling's factor / low / high / original, if given)
              right  retention: S <- decay_h S + k v^T with k scaled by dim^-1/2, o = S^T q, each head
                     divided by its root mean square (no weight), times silu(g h), then `o`
  mlp         a mixture of experts: scores = softmax over all experts of the float32 router logits, the `top`
              largest chosen and divided by their sum + 1e-20; an expert is down(relu(up x)^2); a shared
              expert of the same form for every token, times sigmoid(sg . x)
  output      RMSNorm `final.norm`, `head`, logits times logit_scale

Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.{q,k,v,g,o,a1,a2,a2.b,norm}` or
`l<i>.mix.left.{q,k,v,o}` and `l<i>.mix.right.{q,k,v,g,o}`, `l<i>.mlp.{router,e<j>.up,e<j>.down,shared.up,
shared.down,shared.sg}`, `final.norm`, `head`.  The rank of the decay's projection is A1's first size.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Dict, Optional, Tuple

from ..config.model_config import ConfigError, _require, _typed
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import ModelFamily, register_architecture

DEFAULT_POSITIONS = 1 << 16       # config.json names no longest sequence: what the engine plans its tables for
DEFAULT_DECAY_RANK = 32           # of random weights; a checkpoint's own is read from its tensor


def _opt(raw: Optional[Dict[str, Any]], key: str, typ, where: str):
    return None if not raw or raw.get(key) is None else _typed(raw[key], key, typ, where)


def _obj(raw: Any, what: str, where: str) -> Dict[str, Any]:
    if not isinstance(raw, dict):
        raise ConfigError(f"{where}: {what!r} must be an object")
    return raw


@dataclass(frozen=True)
class RotaryPositions:
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None      # factor, low, high, original

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "RotaryPositions":
        raw = _obj(raw, "rot", where)
        sc = raw.get("scaling")
        scaling = None
        if sc is not None:
            sc = _obj(sc, "rot.scaling", where)
            scaling = tuple(_require(sc, k, float, where) for k in ("factor", "low", "high", "original"))
            if not (scaling[0] > 0 and scaling[3] > 0 and scaling[1] != scaling[2] and scaling[1] > 0 and scaling[2] > 0):
                raise ConfigError(f"{where}: rot.scaling needs positive numbers and low != high")
        r = cls(_require(raw, "dims", int, where), _require(raw, "base", float, where), scaling)
        if r.dims <= 0 or r.dims % 2 or not r.base > 0:
            raise ConfigError(f"{where}: rot.dims must be even and positive, rot.base positive")
        return r

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return out


@dataclass(frozen=True)
class SoftmaxBranch:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotaryPositions]

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "SoftmaxBranch":
        raw = _obj(raw, "left", where)
        dim = _require(raw, "dim", int, where)
        b = cls(_require(raw, "heads", int, where), _require(raw, "kv_heads", int, where), dim,
                _opt(raw, "vdim", int, where) or dim,
                _require(raw, "scale", float, where),
                RotaryPositions.from_dict(raw["rot"], where) if raw.get("rot") is not None else None)
        if min(b.heads, b.kv_heads, b.dim, b.vdim) <= 0 or b.heads % b.kv_heads:
            raise ConfigError(f"{where}: {b.heads} heads of {b.dim}/{b.vdim} on {b.kv_heads} kv heads cannot be run")
        if b.rot is not None and b.rot.dims > b.dim:
            raise ConfigError(f"{where}: {b.rot.dims} rotated dims of a head of {b.dim}")
        return b

    def to_dict(self) -> Dict[str, Any]:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class RetentionBranch:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "RetentionBranch":
        raw = _obj(raw, "right", where)
        decay = raw.get("decay")
        if not isinstance(decay, list):
            raise ConfigError(f"{where}: 'decay' must be a list, one number a head")
        dim = _require(raw, "dim", int, where)
        b = cls(_require(raw, "heads", int, where), dim, _opt(raw, "vdim", int, where) or dim,
                tuple(_typed(d, "decay", float, where) for d in decay))
        if min(b.heads, b.dim, b.vdim) <= 0 or len(b.decay) != b.heads:
            raise ConfigError(f"{where}: {b.heads} heads of {b.dim}/{b.vdim} with {len(b.decay)} decays cannot be run")
        return b

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class ParallelMixer:
    left: SoftmaxBranch
    right: RetentionBranch
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "ParallelMixer":
        raw = _obj(raw, "mixer", where)
        return cls(SoftmaxBranch.from_dict(raw.get("left"), where), RetentionBranch.from_dict(raw.get("right"), where),
                   _require(raw, "left_scale", float, where), _require(raw, "right_scale", float, where))

    def to_dict(self) -> Dict[str, Any]:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class GlaMixer:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = DEFAULT_DECAY_RANK       # no key of config.json: the checkpoint's tensor says it

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> "GlaMixer":
        raw = _obj(raw, "mixer", where)
        dim = _require(raw, "dim", int, where)
        m = cls(_require(raw, "heads", int, where), dim, _opt(raw, "vdim", int, where) or dim, _require(raw, "tau", float, where))
        if min(m.heads, m.dim, m.vdim) <= 0 or not m.tau > 0:
            raise ConfigError(f"{where}: {m.heads} heads of {m.dim}/{m.vdim} with tau {m.tau} cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


@dataclass(frozen=True)
class ExpertsMlp:
    ff: int
    experts: int
    top: int
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, raw: Any, where: str) -> Optional["ExpertsMlp"]:
        if raw is None:
            return None
        raw = _obj(raw, "mlp", where)
        kind = raw.get("kind", "moe")
        if kind != "moe":
            raise ConfigError(f"{where}: unknown mlp kind {kind!r} (moe)")
        m = cls(_require(_obj(raw.get("expert"), "expert", where), "ff", int, where),
                _require(_obj(raw.get("router"), "router", where), "experts", int, where),
                _require(raw["router"], "top", int, where),
                _require(_obj(raw["shared"], "shared", where), "ff", int, where) if raw.get("shared") is not None else None)
        if m.ff <= 0 or not (0 < m.top <= m.experts) or (m.shared_ff is not None and m.shared_ff <= 0):
            raise ConfigError(f"{where}: {m.top} of {m.experts} experts of {m.ff} (shared: {m.shared_ff}) cannot be run")
        return m

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class LilalornLayer:
    type: str                        # "gla" or "parallel"
    mixer: Any                       # GlaMixer or ParallelMixer
    mlp: Optional[ExpertsMlp]
    weights_of: Optional[int] = None


@dataclass(frozen=True)
class LilalornConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    logit_scale: float
    layers: Tuple[LilalornLayer, ...]
    max_positions: int = DEFAULT_POSITIONS
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Lilalorn"

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], where: str = "config.json") -> "LilalornConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where}: 'layers' must be a list of layers")
        out = []
        for i, l in enumerate(layers):
            at = f"{where}: layers[{i}]"
            l = _obj(l, f"layers[{i}]", where)
            kind = _require(l, "type", str, at)
            if kind == "gla":
                mixer = GlaMixer.from_dict(l.get("mixer"), at)
            elif kind == "parallel":
                mixer = ParallelMixer.from_dict(l.get("mixer"), at)
            else:
                raise ConfigError(f"{at}: unknown layer type {kind!r} (gla, parallel)")
            out.append(LilalornLayer(kind, mixer, ExpertsMlp.from_dict(l.get("mlp"), at), _opt(l, "weights_of", int, at)))
        eos = raw.get("eos_token_id")
        cfg = cls(vocab=_require(raw, "vocab", int, where), width=_require(raw, "width", int, where),
                  norm_eps=_require(_obj(raw.get("norm"), "norm", where), "eps", float, where),
                  residual_mult=_opt(raw, "residual_mult", float, where) if raw.get("residual_mult") is not None else 1.0,
                  logit_scale=_opt(raw, "logit_scale", float, where) if raw.get("logit_scale") is not None else 1.0,
                  layers=tuple(out), max_positions=_opt(raw, "max_positions", int, where) or DEFAULT_POSITIONS,
                  eos_token_id=None if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos])),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Lilalorn"])[0]))
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_positions <= 0:
            raise ConfigError(f"{where}: vocab, width and max_positions must be positive")
        for i in range(len(cfg.layers)):
            cfg.owner_of(i, where)
        return cfg

    def owner_of(self, i: int, where: str = "config.json") -> int:
        """The layer whose tensors layer i runs with (itself, unless it says `weights_of`)."""
        seen = {i}
        j = i
        while self.layers[j].weights_of is not None:
            j = self.layers[j].weights_of
            if not (0 <= j < len(self.layers)) or j in seen:
                raise ConfigError(f"{where}: layers[{i}]: weights_of leads to no layer with tensors")
            seen.add(j)
        return j

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            d: Dict[str, Any] = {"type": l.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
            if l.weights_of is not None:
                d["weights_of"] = l.weights_of
            layers.append(d)
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                               "logit_scale": self.logit_scale, "layers": layers}
        if self.max_positions != DEFAULT_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            out["eos_token_id"] = list(self.eos_token_id)
        return out


def _left_spec(cfg: LilalornConfig, b: SoftmaxBranch) -> PartSpec:
    position = None
    if b.rot is not None:
        params: Dict[str, Any] = dict(head_dim=b.dim, rotary_dim=b.rot.dims, theta=b.rot.base, max_positions=cfg.max_positions)
        if b.rot.scaling is not None:
            factor, low, high, original = b.rot.scaling
            params["scaling"] = dict(kind="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high, original=original)
        position = PartSpec("rope", params)
    return PartSpec("attention", dict(
        hidden_size=cfg.width, num_heads=b.heads, num_kv_heads=b.kv_heads, head_dim=b.dim, value_dim=b.vdim, bias=False,
        qk_norm=False, window=None, position=position, scale=b.scale, names={"q": "q", "k": "k", "v": "v", "o": "o"}))


def _mixer_spec(cfg: LilalornConfig, l: LilalornLayer) -> PartSpec:
    m = l.mixer
    if l.type == "gla":
        return PartSpec("gated_linear_attention", dict(
            hidden_size=cfg.width, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, tau=m.tau, decay_rank=m.decay_rank,
            norm_eps=cfg.norm_eps))
    right = PartSpec("retention", dict(hidden_size=cfg.width, num_heads=m.right.heads, key_dim=m.right.dim,
                                       value_dim=m.right.vdim, decay=m.right.decay, norm_eps=cfg.norm_eps))
    return PartSpec("parallel", dict(branches=(("left", m.left_scale, _left_spec(cfg, m.left)),
                                               ("right", m.right_scale, right))))


def _mlp_spec(cfg: LilalornConfig, mlp: ExpertsMlp) -> PartSpec:
    params: Dict[str, Any] = dict(
        hidden_size=cfg.width, intermediate_size=mlp.ff, num_experts=mlp.experts, top=mlp.top, router_bias=False,
        activation="relu2", gated=False, scores="all",
        names={"router": "router", "up": "e{i}.up", "down": "e{i}.down", "shared_up": "shared.up",
               "shared_down": "shared.down", "shared_open": "shared.sg"})
    if mlp.shared_ff is not None:
        params["shared"] = dict(intermediate_size=mlp.shared_ff, activation="relu2", gated=False, gate=True)
    return PartSpec("routed_experts", params)


def lilalorn_spec(cfg: LilalornConfig) -> ModelSpec:
    own = [i for i, l in enumerate(cfg.layers) if l.weights_of is None]
    index = {i: n for n, i in enumerate(own)}                  # config layer -> place in the spec's layers
    layers = []
    for i in own:
        l = cfg.layers[i]
        norms = {"norm1": PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm1"))}
        if l.mlp is not None:
            norms["norm2"] = PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name=f"l{i}.norm2"))
        layers.append(LayerSpec(prefix=f"l{i}", block="prenorm", mixer=_mixer_spec(cfg, l),
                                feed_forward=None if l.mlp is None else _mlp_spec(cfg, l.mlp), norms=norms,
                                mixer_name="mix", feed_forward_name="mlp",
                                block_params={"residual_scale": cfg.residual_mult}))
    schedule, next_id = [], len(own)
    for i, l in enumerate(cfg.layers):
        if l.weights_of is None:
            schedule.append(ScheduleEntry(index[i]))
        else:                                                   # another layer's tensors, a cache and state of its own
            schedule.append(ScheduleEntry(index[cfg.owner_of(i)], cache_id=next_id))
            next_id += 1
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=cfg.width, max_positions=cfg.max_positions,
        embedding=PartSpec("embedding", dict(name="embed", vocab_size=cfg.vocab, dim=cfg.width)),
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=PartSpec("rmsnorm", dict(dim=cfg.width, eps=cfg.norm_eps, name="final.norm")),
        head=PartSpec("lm_head", dict(name="head", tied=False, vocab_size=cfg.vocab, dim=cfg.width, scale=cfg.logit_scale)),
        eos_token_ids=tuple(cfg.eos_token_id or ()))


def lilalorn_spec_for(cfg: LilalornConfig, tensor_names) -> ModelSpec:
    """The spec for a checkpoint: the rank of each gla layer's decay projection is its `a1` tensor's first size."""
    shape_of = getattr(tensor_names, "shape_of", None)
    names = set(tensor_names)
    if shape_of is not None:
        layers = list(cfg.layers)
        for i, l in enumerate(layers):
            name = f"l{i}.mix.a1"
            if l.type == "gla" and l.weights_of is None and name in names:
                layers[i] = replace(l, mixer=replace(l.mixer, decay_rank=int(shape_of(name)[0])))
        for i, l in enumerate(layers):
            if l.type == "gla" and l.weights_of is not None:
                layers[i] = replace(l, mixer=layers[cfg.owner_of(i)].mixer)
        cfg = replace(cfg, layers=tuple(layers))
    return lilalorn_spec(cfg)


LILALORN = ModelFamily("lilalorn", LilalornConfig, lilalorn_spec, build_spec_for=lilalorn_spec_for)
register_architecture("Lilalorn", LILALORN)
