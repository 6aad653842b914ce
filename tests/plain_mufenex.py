"""Plain, slow Mufenex on the CPU: whole sequences, no cache, one function per mechanism, torch
tensor arithmetic in float32 or float64 only.  It shares no code with xinfer_amd: it parses
config.json itself and reads the weights with the `safetensors` package.

Notation: x [n, width] is the residual stream of a sequence of n tokens at positions 0..n-1;
`W[name]` a tensor of the checkpoint; linear weights are [out, in] and applied as x @ W^T.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def read_weights(model_dir: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            out[k] = f.get_tensor(k).to(dtype)
    return out


# ---- mechanisms, one function each ---------------------------------------------------------
def rms_norm(x: torch.Tensor, eps: float, w: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis (eps inside the root), times w if given."""
    y = x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def sinusoid_positions(n: int, width: int, dtype, first: int = 0, base: float = 10000.0) -> torch.Tensor:
    """Row p: entry 2i = sin(p * base^(-2i / width)), entry 2i + 1 = cos of the same angle."""
    i = torch.arange((width + 1) // 2, dtype=dtype)
    freq = torch.tensor(base, dtype=dtype) ** (-2.0 * i / width)
    ang = torch.arange(first, first + n, dtype=dtype)[:, None] * freq[None, :]
    out = torch.zeros(n, 2 * freq.numel(), dtype=dtype)
    out[:, 0::2] = ang.sin()
    out[:, 1::2] = ang.cos()
    return out[:, :width]


def embed(tokens: List[int], table: torch.Tensor, scale: float) -> torch.Tensor:
    x = table[torch.tensor(tokens, dtype=torch.long)] * scale
    return x + sinusoid_positions(len(tokens), table.shape[1], table.dtype)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def head_slope(h: int, heads: int) -> float:
    return 2.0 ** (-8.0 * (h + 1) / heads)


def visible(n_q: int, n_k: int, first_q: int, window: Optional[int]) -> torch.Tensor:
    """[n_q, n_k] True where query at position first_q + a sees key at position b: 0 <= i - j (< window)."""
    i = torch.arange(first_q, first_q + n_q)[:, None]
    j = torch.arange(n_k)[None, :]
    ok = (i - j) >= 0
    if window:
        ok &= (i - j) < window
    return ok


def scores(q: torch.Tensor, k: torch.Tensor, scale: float, softcap: Optional[float], slope: Optional[float],
           window: Optional[int], first_q: int = 0) -> torch.Tensor:
    """One head: q [n_q, d] at positions first_q.., k [n_k, d] at positions 0..: softmax weights [n_q, n_k]."""
    s = (q @ k.T) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if slope is not None:
        i = torch.arange(first_q, first_q + q.shape[0], dtype=q.dtype)[:, None]
        j = torch.arange(k.shape[0], dtype=q.dtype)[None, :]
        s = s - slope * (i - j)
    s = s.masked_fill(~visible(q.shape[0], k.shape[0], first_q, window), float("-inf"))
    return torch.softmax(s, dim=-1)


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, softcap: Optional[float],
           window: Optional[int], biased: bool = True, first_q: int = 0) -> torch.Tensor:
    """q [n_q, H, d], k [n_k, G, d], v [n_k, G, dv] -> [n_q, H * dv]; query head h reads kv head h // (H / G)."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        p = scores(q[:, h], k[:, g], scale, softcap, head_slope(h, H) if biased else None, window, first_q)
        out[:, h] = p @ v[:, g]
    return out.reshape(n, -1)


def blend_values(v: torch.Tensor, v_first: torch.Tensor, lam: torch.Tensor) -> torch.Tensor:
    return (1.0 - lam) * v + lam * v_first


def attention_mixer(x: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, v_first):
    """Returns (output [n, width], the values before blending)."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim") or m["dim"]
    n = x.shape[0]
    q = rms_norm(x @ W[p + "q"].T, eps, W[p + "q.norm"])
    k = rms_norm(x @ W[p + "k"].T, eps, W[p + "k.norm"])
    v = v_own = x @ W[p + "v"].T
    if v_first is not None:
        v = blend_values(v, v_first, W[p + "vmix"])
    window = (m.get("mask") or {}).get("size")
    a = attend(q.view(n, H, d), k.view(n, G, d), v.view(n, G, dv), m["scale"], m.get("softcap"), window)
    return a @ W[p + "o"].T, v_own


def dense_ff(x: torch.Tensor, W: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (gelu_tanh(x @ W[p + "gate"].T) * (x @ W[p + "up"].T)) @ W[p + "down"].T


def route(x: torch.Tensor, W: Dict[str, torch.Tensor], p: str, top: int):
    """(chosen experts [n, top] in descending order of their logits, weights [n, top])."""
    z = x @ W[p + "router"].T + W[p + "router.b"]
    val, idx = z.topk(top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def experts_ff(x: torch.Tensor, W: Dict[str, torch.Tensor], p: str, ml: dict) -> torch.Tensor:
    idx, wt = route(x, W, p, ml["router"]["top"])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for r in range(idx.shape[1]):
            e = f"{p}e{int(idx[t, r])}."
            out[t] += wt[t, r] * ((silu(W[e + "gate"] @ x[t]) * (W[e + "up"] @ x[t])) @ W[e + "down"].T)
    return out


class PlainMufenex:
    def __init__(self, model_dir: str, dtype=torch.float32):
        self.c = read_config(model_dir)
        self.W = read_weights(model_dir, dtype)
        self.dtype = dtype

    def stream(self, tokens: List[int]) -> List[torch.Tensor]:
        """The residual stream after the embedding and after every layer."""
        c, W = self.c, self.W
        eps = c["norm"]["eps"]
        x = embed(tokens, W["embed"], (c.get("embedding") or {}).get("scale", 1.0))
        out = [x]
        v_first = None
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            m = layer["mixer"]
            mixing = bool(m.get("v_mix"))
            a, v_own = attention_mixer(x, W, p + "mix.", m, eps, v_first if mixing else None)
            if mixing and v_first is None:
                v_first = v_own
            x = x + rms_norm(a, eps, W[p + "norm1"])
            ml = layer.get("mlp")
            if ml is not None:
                f = dense_ff(x, W, p + "mlp.") if ml["kind"] == "dense" else experts_ff(x, W, p + "mlp.", ml)
                x = x + rms_norm(f, eps, W[p + "norm2"])
            out.append(x)
        return out

    def logits(self, tokens: List[int]) -> torch.Tensor:
        c, W = self.c, self.W
        x = rms_norm(self.stream(tokens)[-1], c["norm"]["eps"], W["final.norm"])
        lg = x @ W["head"].T
        cap = c.get("logit_softcap")
        return cap * torch.tanh(lg / cap) if cap else lg

    def greedy(self, prompt: List[int], n: int) -> List[int]:
        ids = list(prompt)
        for _ in range(n):
            ids.append(int(self.logits(ids)[-1].argmax()))
        return ids[len(prompt):]
