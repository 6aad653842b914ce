"""A plain, slow Lilalorn written from the design's equations: one function a mechanism, every token of a
sequence at once or one by one, no cache, no batching, no kernels.  It reads a model folder by itself
(config.json, model.safetensors through the safetensors library) and shares no code with the engine.

Notation: x the residual stream [T, width], h a sublayer's input, p a token's position (from 0).
"""
import json
import math
import os

import torch
from safetensors import safe_open


# ---- norms and small functions ---------------------------------------------------------------------
def rms_norm(x, eps, w=None):
    """x / sqrt(mean(x^2) + eps) over the last axis, times w if given."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z):
    return z * torch.sigmoid(z)


def relu_squared(z):
    return torch.relu(z) ** 2


# ---- rotary positions --------------------------------------------------------------------------------
def rotary_frequencies(rot, dtype=torch.float64):
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` (factor, low, high, original) a frequency whose
    wavelength l = 2 pi / f is shorter than original / high stays, one longer than original / low is divided
    by factor, and between the two both are blended by s = (original / l - low) / (high - low)."""
    d = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / d) for i in range(d // 2)], dtype=dtype)
    sc = rot.get("scaling")
    if not sc:
        return f
    out = []
    for fi in f.tolist():
        l = 2 * math.pi / fi
        if l < sc["original"] / sc["high"]:
            out.append(fi)
        elif l > sc["original"] / sc["low"]:
            out.append(fi / sc["factor"])
        else:
            s = (sc["original"] / l - sc["low"]) / (sc["high"] - sc["low"])
            out.append((1 - s) * fi / sc["factor"] + s * fi)
    return torch.tensor(out, dtype=dtype)


def rotate(x, rot, positions):
    """x [T, heads, dim]: dims i and i + dims / 2 of every head, i < dims / 2, turn by the angle p f_i:
    (u, v) -> (u cos - v sin, v cos + u sin); dims from rot.dims on pass unchanged."""
    if rot is None:
        return x
    d = rot["dims"]
    ang = positions.to(x.dtype)[:, None] * rotary_frequencies(rot, x.dtype)[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    u, v = x[..., :d // 2], x[..., d // 2:d]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., d:]], dim=-1)


# ---- the three mixers' cores -----------------------------------------------------------------------------
def softmax_attention(q, k, v, scale):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads kv head h // (H / G); token i sees every
    j <= i; softmax of (q . k) * scale.  Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def decaying_state(q, k, v, a, state=None):
    """Per head a matrix S [dk, dv], from zeros (or `state`): S <- diag(a_t) S + k_t v_t^T, o_t = S^T q_t.
    q, k, a [T, H, dk], v [T, H, dv].  Returns (o [T, H, dv], the last S)."""
    T, H, dk = q.shape
    S = torch.zeros(H, dk, v.shape[-1], dtype=q.dtype) if state is None else state.clone()
    out = []
    for t in range(T):
        S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hkv,hk->hv", S, q[t]))
    return torch.stack(out), S


# ---- mixture of experts -----------------------------------------------------------------------------------
def router_weights(z, top):
    """z [T, E] router logits.  Scores = softmax over all experts; the `top` largest are chosen and divided by
    their sum + 1e-20.  Returns (indices [T, top], weights [T, top])."""
    s = torch.softmax(z, dim=-1)
    val, idx = s.topk(top, dim=-1)
    return idx, val / (val.sum(dim=-1, keepdim=True) + 1e-20)


def expert(h, up, down):
    return relu_squared(h @ up.T) @ down.T


class PlainLilalorn:
    def __init__(self, model_dir, dtype=torch.float64):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.c = json.load(f)
        self.dtype = dtype
        self.W = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.W[name] = f.get_tensor(name).to(dtype)
        self.eps = self.c["norm"]["eps"]

    # -- mixers ------------------------------------------------------------------------------------------
    def left(self, p, m, h, positions):
        T = h.shape[0]
        q = (h @ self.W[p + ".q"].T).view(T, m["heads"], m["dim"])
        k = (h @ self.W[p + ".k"].T).view(T, m["kv_heads"], m["dim"])
        v = (h @ self.W[p + ".v"].T).view(T, m["kv_heads"], m.get("vdim", m["dim"]))
        q, k = rotate(q, m.get("rot"), positions), rotate(k, m.get("rot"), positions)
        return softmax_attention(q, k, v, m["scale"]).reshape(T, -1) @ self.W[p + ".o"].T

    def right(self, p, m, h):
        T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
        q = (h @ self.W[p + ".q"].T).view(T, H, dk)
        k = (h @ self.W[p + ".k"].T).view(T, H, dk) * dk ** -0.5
        v = (h @ self.W[p + ".v"].T).view(T, H, dv)
        a = torch.tensor(m["decay"], dtype=self.dtype)[None, :, None].expand(T, H, dk)
        o, _ = decaying_state(q, k, v, a)
        o = rms_norm(o, self.eps).reshape(T, H * dv)
        return (o * silu(h @ self.W[p + ".g"].T)) @ self.W[p + ".o"].T

    def gla(self, p, m, h):
        T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
        q = (h @ self.W[p + ".q"].T).view(T, H, dk) * dk ** -0.5
        k = (h @ self.W[p + ".k"].T).view(T, H, dk)
        v = (h @ self.W[p + ".v"].T).view(T, H, dv)
        z = (h @ self.W[p + ".a1"].T) @ self.W[p + ".a2"].T + self.W[p + ".a2.b"]
        a = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, dk)
        o, _ = decaying_state(q, k, v, a)
        o = rms_norm(o, self.eps, self.W[p + ".norm"]).reshape(T, H * dv)
        return (o * silu(h @ self.W[p + ".g"].T)) @ self.W[p + ".o"].T

    def mixer(self, p, layer, h, positions):
        m = layer["mixer"]
        if layer["type"] == "gla":
            return self.gla(p + ".mix", m, h)
        return (m["left_scale"] * self.left(p + ".mix.left", m["left"], h, positions)
                + m["right_scale"] * self.right(p + ".mix.right", m["right"], h))

    # -- feed-forward -----------------------------------------------------------------------------------------
    def router_logits(self, p, h):
        return h @ self.W[p + ".router"].T

    def feed_forward(self, p, ml, h):
        idx, wt = router_weights(self.router_logits(p, h), ml["router"]["top"])
        out = torch.zeros_like(h)
        for t in range(h.shape[0]):
            for r in range(idx.shape[1]):
                e = int(idx[t, r])
                out[t] += wt[t, r] * expert(h[t], self.W[f"{p}.e{e}.up"], self.W[f"{p}.e{e}.down"])
        if ml.get("shared"):
            out = out + expert(h, self.W[p + ".shared.up"], self.W[p + ".shared.down"]) * torch.sigmoid(h @ self.W[p + ".shared.sg"].T)
        return out

    # -- the model ---------------------------------------------------------------------------------------------
    def tensors_of(self, i):
        """The layer whose tensors layer i runs with."""
        while self.c["layers"][i].get("weights_of") is not None:
            i = self.c["layers"][i]["weights_of"]
        return i

    def stream(self, tokens):
        """The residual stream entering every layer, and after the last one: a list of [T, width]."""
        x = self.W["embed"][torch.tensor(tokens)]
        positions = torch.arange(len(tokens))
        m = self.c.get("residual_mult", 1.0)
        out = [x]
        for i, layer in enumerate(self.c["layers"]):
            p = f"l{self.tensors_of(i)}"
            x = x + m * self.mixer(p, layer, rms_norm(x, self.eps, self.W[p + ".norm1"]), positions)
            if layer.get("mlp") is not None:
                x = x + m * self.feed_forward(p + ".mlp", layer["mlp"], rms_norm(x, self.eps, self.W[p + ".norm2"]))
            out.append(x)
        return out

    def logits(self, tokens):
        x = self.stream(tokens)[-1]
        return (rms_norm(x, self.eps, self.W["final.norm"]) @ self.W["head"].T) * self.c.get("logit_scale", 1.0)

    def greedy(self, prompt, n):
        ids, out = list(prompt), []
        for _ in range(n):
            t = int(self.logits(ids)[-1].argmax())
            out.append(t)
            ids.append(t)
        return out
