"""Small Mufenex configurations for tests, and the maker of their model folders.

P: three layers that differ in everything: two windows (two cache groups) and a layer that sees
every key, value heads wider and narrower than the key heads, groups of 3, 3 and 1 query heads a
kv head, a dense, a routed and no feed-forward, a layer without soft cap, blended values in all.
Q: the values that other models happen to make equal or 1: value size = key size, one kv head
and as many kv heads as heads, one chosen expert, no embedding scale, no soft cap on the logits,
a layer that blends no values before the ones that do (so the first blending layer is not
layer 0), a width that is no multiple of 8.
S: nothing blended anywhere, no cap on any score, windows of 1 and 2 keys and one wider than any request, all
experts chosen, a first layer without feed-forward, head sizes in eights that are no multiple of 16.
O: sizes in no kernel's favourite multiples (width 50, heads of 12, 20 and 10, 18 and 34 hidden features): every
vectorized form steps aside for its plain one, in bfloat16 too.
R: real-looking head sizes (64 and 128) with few layers, for the matrix-core kernels.

Random weights would leave the router's choice to close calls (bfloat16 rounds the stream, and two
experts' logits often lie closer than that): `make_model` therefore writes weights in which the
choice is decided by a few columns of the stream that nothing but the embedding writes to: the
last `MARKERS` columns hold +-MARK by the bits of the token's id (the sinusoid is nearly constant
there), the norms' weights are zero there so that no branch adds to them, and the routers read
those columns alone.  Which experts a token takes still differs from token to token.
"""
import json
import os

import torch

MARKERS = 4
MARK = 6.0
MARGIN = 0.3         # least distance between the last chosen logit and the first left out


def _mixer(heads, kv_heads, dim, vdim, scale, softcap=None, window=None, v_mix=True):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, v_mix=v_mix)
    if softcap is not None:
        m["softcap"] = softcap
    if window is not None:
        m["mask"] = {"size": window}
    return m


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


MODELS = {
    "P": dict(
        config={"architecture": "Mufenex", "vocab": 331, "width": 96, "embedding": {"scale": 0.7},
                "norm": {"eps": 1e-5}, "logit_softcap": 9.0, "layers": [
                    _layer(_mixer(6, 2, 16, 24, 0.3, softcap=20.0, window=12), {"kind": "dense", "ff": 160}),
                    _layer(_mixer(6, 2, 32, 24, 0.2, softcap=None, window=21), _moe(48, 5, 2)),
                    _layer(_mixer(4, 4, 16, 12, 0.25, softcap=35.0, window=None), None)]},
        seed=11, linear_std=0.08, norm_std=0.1, page_size=16),
    "Q": dict(
        config={"architecture": "Mufenex", "vocab": 257, "width": 100, "norm": {"eps": 1e-6}, "layers": [
            _layer(_mixer(2, 1, 16, 16, 0.25, softcap=15.0, window=9, v_mix=False), _moe(24, 3, 1)),
            _layer(_mixer(5, 5, 16, 16, 0.25, softcap=15.0, window=9), {"kind": "dense", "ff": 72}),
            _layer(_mixer(5, 1, 32, 80, 0.18, softcap=15.0, window=17), _moe(40, 7, 3)),
            _layer(_mixer(1, 1, 48, 80, 0.15, softcap=50.0, window=9), {"kind": "dense", "ff": 56})]},
        seed=12, linear_std=0.1, norm_std=0.2, page_size=8),
    "S": dict(
        config={"architecture": "Mufenex", "vocab": 190, "width": 72, "embedding": {"scale": 1.5}, "norm": {"eps": 1e-6},
                "logit_softcap": 20.0, "layers": [
                    _layer(_mixer(6, 3, 24, 40, 0.2, window=1, v_mix=False), None),
                    _layer(_mixer(3, 3, 8, 8, 0.35, window=200, v_mix=False), _moe(16, 3, 3)),
                    _layer(_mixer(2, 2, 40, 24, 0.16, window=2, v_mix=False), {"kind": "dense", "ff": 40})]},
        seed=14, linear_std=0.1, norm_std=0.15, page_size=8),
    "O": dict(
        config={"architecture": "Mufenex", "vocab": 131, "width": 50, "embedding": {"scale": 0.9}, "norm": {"eps": 1e-5},
                "logit_softcap": 12.0, "layers": [
                    _layer(_mixer(3, 1, 12, 20, 0.3, softcap=25.0, window=7), _moe(18, 4, 2)),
                    _layer(_mixer(2, 2, 20, 10, 0.22, softcap=25.0, window=30), {"kind": "dense", "ff": 34})]},
        seed=15, linear_std=0.1, norm_std=0.1, page_size=8),
    "R": dict(
        config={"architecture": "Mufenex", "vocab": 409, "width": 512, "embedding": {"scale": 2.0},
                "norm": {"eps": 1e-6}, "logit_softcap": 30.0, "layers": [
                    _layer(_mixer(8, 2, 64, 128, 0.125, softcap=30.0, window=100), _moe(128, 8, 2)),
                    _layer(_mixer(4, 4, 128, 64, 0.09, softcap=30.0, window=300), {"kind": "dense", "ff": 768})]},
        seed=13, linear_std=0.04, norm_std=0.1, page_size=64),
}


def make_model(model_dir, name):
    """Writes the folder of configuration `name` (random weights, decisive routers); returns the folder."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    from xinfer_amd.weights import write_random_model
    t = MODELS[name]
    write_random_model(model_dir, t["config"], t["seed"], t["linear_std"], t["norm_std"])
    path = os.path.join(model_dir, "model.safetensors")
    W = {}
    with safe_open(path, framework="pt") as f:
        for k in f.keys():
            W[k] = f.get_tensor(k).clone()
    c = t["config"]
    width = c["width"]
    cols = list(range(width - MARKERS, width))
    scale = (c.get("embedding") or {}).get("scale", 1.0)
    ids = torch.arange(c["vocab"])
    for b, col in enumerate(cols):
        W["embed"][:, col] = (((ids >> b) & 1).float() * 2 - 1) * (MARK / scale)
    g = torch.Generator().manual_seed(t["seed"])
    for i, layer in enumerate(c["layers"]):
        for n in ("norm1", "norm2"):
            if f"l{i}.{n}" in W:
                W[f"l{i}.{n}"][cols] = 0
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            top, experts = layer["mlp"]["router"]["top"], layer["mlp"]["router"]["experts"]
            # the 2^MARKERS patterns the routers can see (sines there are about 0, cosines about 1)
            pats = torch.tensor([[(1.0 if (p >> b) & 1 else -1.0) * MARK + (col % 2) for b, col in enumerate(cols)]
                                 for p in range(1 << MARKERS)])
            for _ in range(2000):          # until every pattern's choice is clear by MARGIN
                rw = (torch.randn(experts, MARKERS, generator=g) * 0.5).to(torch.bfloat16).float()
                rb = (torch.randn(experts, generator=g) * 0.5).to(torch.bfloat16).float()
                z = (pats @ rw.T + rb).sort(dim=-1, descending=True).values
                if top == experts or float((z[:, top - 1] - z[:, top]).min()) >= MARGIN:
                    break
            else:
                raise RuntimeError("no decisive router found")
            r = torch.zeros_like(W[f"l{i}.mlp.router"], dtype=torch.float32)
            r[:, cols] = rw
            W[f"l{i}.mlp.router"] = r.to(torch.bfloat16)
            W[f"l{i}.mlp.router.b"] = rb.to(torch.bfloat16)
    save_file({k: v.contiguous() for k, v in W.items()}, path)
    return model_dir


def router_margin(model_dir, tokens):
    """The least distance, over a sequence's tokens and the model's routers, between the last chosen
    expert's logit and the first one left out (float64, plain implementation)."""
    import plain_mufenex as plain
    pm = plain.PlainMufenex(model_dir, torch.float64)
    streams = pm.stream(tokens)
    least = float("inf")
    for i, layer in enumerate(pm.c["layers"]):
        ml = layer["mlp"]
        if not ml or ml["kind"] != "moe" or ml["router"]["top"] == ml["router"]["experts"]:
            continue
        # the routers read the marker columns alone, which no branch changes: any layer's stream will do
        z = streams[i] @ pm.W[f"l{i}.mlp.router"].T + pm.W[f"l{i}.mlp.router.b"]
        top = ml["router"]["top"]
        val, _ = z.topk(top + 1, dim=-1)
        least = min(least, float((val[:, top - 1] - val[:, top]).min()))
    return least
