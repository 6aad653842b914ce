"""Block arrangements.

"prenorm": x -> norm -> mixer -> (+x, norm) -> feed-forward -> (+r)
(reference: Qwen3DecoderLayer::forward, /root/reference/src/models/qwen3.rs:108-134).
Each residual add is carried out by the norm kernel that follows it: a block hands on
the stream with its feed-forward output still pending, and the next block's first
norm (or the model's final norm) adds it.  With the block parameter `residual_scale` m the
stream gets m times each branch, x <- x + m * mixer(norm(x)), then x <- x + m * ff(norm(x)); a layer
without a feed-forward ends after the first of the two.

"branchnorm": x <- x + norm1(mixer(x)); x <- x + norm2(ff(x)): the sublayers read the stream
itself and their OUTPUT is normed; a layer may have no feed-forward.  The norm, the add and
the rounding of the new stream for the next sublayer are one kernel (`Norm.forward_branch`).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..config.spec import LayerSpec
from ..weights.store import TensorDecl, WeightStore
from .base import (Block, Folded, KVNeed, LayerCache, NormSink, StateNeed, StepContext, Stream,
                   feed_forward_class, mixer_class, norm_class, register_block)

@register_block("prenorm")
class PreNormBlock(Block):
    """Runs two norms: `layer.norms` names the one before the mixer first, then the one before
    the feed-forward.  Every tensor name comes from the `LayerSpec`."""

    def __init__(self, layer: LayerSpec, dtype: torch.dtype):
        super().__init__(layer, dtype)
        self.mixer = mixer_class(layer.mixer.kind)(layer.mixer, dtype)
        self.ffn = (feed_forward_class(layer.feed_forward.kind)(layer.feed_forward, dtype)
                    if layer.feed_forward is not None else None)
        self.scale = float(layer.block_params.get("residual_scale", 1.0))
        items = layer.norm_items(2 if self.ffn is not None else 1)
        self._name1, n1 = items[0]
        self.norm1 = norm_class(n1.kind)(n1, dtype)
        self._name2, self.norm2 = None, None
        if self.ffn is not None:
            self._name2, n2 = items[1]
            self.norm2 = norm_class(n2.kind)(n2, dtype)
        # a norm rides on the products around it only where the stream gets the plain sum
        self.folds = self.scale == 1.0 and self.ffn is not None

    @classmethod
    def declare(cls, layer: LayerSpec) -> List[TensorDecl]:
        p = layer.prefix
        out = mixer_class(layer.mixer.kind).declare(layer.mixer, f"{p}.{layer.mixer_name}")
        if layer.feed_forward is not None:
            out += feed_forward_class(layer.feed_forward.kind).declare(layer.feed_forward, f"{p}.{layer.feed_forward_name}")
        for name, n in layer.norm_items(2 if layer.feed_forward is not None else 1):
            out += norm_class(n.kind).declare(n, f"{p}.{name}")
        return out

    def load(self, store: WeightStore, device) -> None:
        p = self.layer.prefix
        self.mixer.load(store, f"{p}.{self.layer.mixer_name}", device)
        self.norm1.load(store, f"{p}.{self._name1}", device)
        if self.ffn is not None:
            self.ffn.load(store, f"{p}.{self.layer.feed_forward_name}", device)
            self.norm2.load(store, f"{p}.{self._name2}", device)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer, self.ffn, self.norm1, self.norm2) if p is not None)

    def cache_need(self) -> Optional[KVNeed]:
        return self.mixer.cache_need()

    def state_need(self) -> Optional[StateNeed]:
        return self.mixer.state_need()

    # ---- folding norms into the products around them (parts.base.Folded) ---------------------
    # `folds` (set per block): `forward` takes `next_norm` and a stream with `folded`

    def first_norm(self):
        """The norm that a block before this one may half do, or None."""
        return self.norm1 if (self.norm1.foldable and self.mixer.takes_folded) else None

    def forward(self, stream: Stream, ctx: StepContext, cache: LayerCache, next_norm=None) -> Stream:
        """`next_norm`: the first norm of the block that runs next, if that block lets this
        one's feed-forward half do it."""
        if not self.folds:
            return self._forward_scaled(stream, ctx, cache)
        if stream.folded is not None:
            if stream.folded.norm is not self.norm1:
                raise RuntimeError("the stream carries a half-done norm of another block")
            h = stream.folded
        elif stream.pending_scale != 1.0:
            h = self.norm1.forward(stream.resid, stream.pending, self.dtype, add_scale=stream.pending_scale)
        else:
            h = self.norm1.forward(stream.resid, stream.pending, self.dtype)
        if self.mixer.takes_sink and self.ffn.takes_folded and self.norm2.foldable:
            a = self.mixer.forward(h, ctx, cache, sink=NormSink(stream.resid, self.norm2))
        else:
            a = self.mixer.forward(h, ctx, cache)
        h2 = a if isinstance(a, Folded) else self.norm2.forward(stream.resid, a, self.dtype)
        if next_norm is not None and self.ffn.takes_sink:
            m = self.ffn.forward(h2, ctx, sink=NormSink(stream.resid, next_norm))
        else:
            m = self.ffn.forward(h2, ctx)
        if isinstance(m, Folded):
            return Stream(stream.resid, None, m)
        return Stream(stream.resid, m)

    def _forward_scaled(self, stream: Stream, ctx: StepContext, cache: LayerCache) -> Stream:
        """The step with a factor on the branches, or without a feed-forward: every add is done by the norm
        kernel that follows it, with its factor."""
        if stream.folded is not None:
            raise RuntimeError("the stream carries a half-done norm of another block")
        resid = stream.resid

        def normed(norm, add, scale):
            if add is not None and scale != 1.0:
                return norm.forward(resid, add, self.dtype, add_scale=scale)
            return norm.forward(resid, add, self.dtype)

        a = self.mixer.forward(normed(self.norm1, stream.pending, stream.pending_scale), ctx, cache)
        if self.ffn is None:
            return Stream(resid, a, pending_scale=self.scale)
        m = self.ffn.forward(normed(self.norm2, a, self.scale), ctx)
        return Stream(resid, m, pending_scale=self.scale)


@register_block("branchnorm")
class BranchNormBlock(Block):
    """`layer.norms` names the norm of the mixer's output first, then the one of the feed-forward's
    output (absent if the layer has no feed-forward)."""

    def __init__(self, layer: LayerSpec, dtype: torch.dtype):
        super().__init__(layer, dtype)
        self.mixer = mixer_class(layer.mixer.kind)(layer.mixer, dtype)
        self.ffn = (feed_forward_class(layer.feed_forward.kind)(layer.feed_forward, dtype)
                    if layer.feed_forward is not None else None)
        items = layer.norm_items(2 if self.ffn is not None else 1)
        self._names = [n for n, _ in items]
        self.norms = [norm_class(n.kind)(n, dtype) for _, n in items]

    @classmethod
    def declare(cls, layer: LayerSpec) -> List[TensorDecl]:
        p = layer.prefix
        out = mixer_class(layer.mixer.kind).declare(layer.mixer, f"{p}.{layer.mixer_name}")
        if layer.feed_forward is not None:
            out += feed_forward_class(layer.feed_forward.kind).declare(layer.feed_forward, f"{p}.{layer.feed_forward_name}")
        for name, n in layer.norm_items(2 if layer.feed_forward is not None else 1):
            out += norm_class(n.kind).declare(n, f"{p}.{name}")
        return out

    def load(self, store: WeightStore, device) -> None:
        p = self.layer.prefix
        self.mixer.load(store, f"{p}.{self.layer.mixer_name}", device)
        if self.ffn is not None:
            self.ffn.load(store, f"{p}.{self.layer.feed_forward_name}", device)
        for name, norm in zip(self._names, self.norms):
            norm.load(store, f"{p}.{name}", device)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer, *self.norms, *(() if self.ffn is None else (self.ffn,))))

    def cache_need(self) -> Optional[KVNeed]:
        return self.mixer.cache_need()

    def state_need(self) -> Optional[StateNeed]:
        return self.mixer.state_need()

    def forward(self, stream: Stream, ctx: StepContext, cache: LayerCache) -> Stream:
        resid = stream.resid
        if stream.folded is not None:
            raise RuntimeError("the stream carries a half-done norm of another block")
        rows_dtype = None if self.dtype == torch.float32 else self.dtype       # float32: the stream is its own rows
        x = stream.rows
        if stream.pending is not None and stream.pending_scale != 1.0:
            raise NotImplementedError("a branch with a factor is left to a block that norms its sublayers' outputs")
        if stream.pending is not None:        # a block of another arrangement left its last branch to be added
            x = kernels.rmsnorm_add(resid, stream.pending, None, 0.0, rows_dtype)
        if rows_dtype is None:
            x = resid
        elif x is None:                       # a stream that came without its rounding (another embedding kind)
            x = resid.to(self.dtype)
        a = self.mixer.forward(x, ctx, cache)
        x = self.norms[0].forward_branch(resid, a, rows_dtype)
        if self.ffn is not None:
            m = self.ffn.forward(x if rows_dtype is not None else resid, ctx)
            x = self.norms[1].forward_branch(resid, m, rows_dtype)
        return Stream(resid, None, None, rows=x)
