"""Small Lilalorn configurations for tests, and the maker of their model folders.

A: both layer types, the orders "parallel, gla" and back, two layers that run with another layer's tensors (one of each
   type), a layer without feed-forward, 2 kv heads for 6 query heads, fewer rotated dims than the head has, value heads
   wider than key heads on the left and narrower on the right, other head counts left and right, frequency scaling
   whose bands all occur, a factor on the branches and on the logits.
B: the values that another model may make equal or 1: value size = key size everywhere (the attention then takes the
   kernels of the plain form), as many kv heads as heads, every dim rotated, no frequency scaling, one chosen expert,
   no shared expert in one layer, factors of 1, tau 1, a gla layer first, decays of 1 and near 0, one head.
O: sizes in no kernel's favourite multiples (width 50, heads of 12, 20 and 10, 18 hidden features, 6 rotated dims of 12,
   a decay projection of rank 5): every vectorized form steps aside for its plain one, in bfloat16 too.
G: layers of one type only, the one that keeps no pages: requests have states and lengths, and no cache to read.
R: real-looking head sizes (64 and 128, states of 128 by 256) with few layers and pages of 64, for the matrix-core
   kernels, and key heads of more than 128 channels for the state's widest form.

Random routers would leave some token's choice of experts to a difference that bfloat16 does not keep: `make_model`
writes weights in which the choice is decided by a few columns of the stream that only the embedding writes to: the
last MARKERS columns hold +-MARK by the bits of the token's id, every product that adds to the stream has zero rows
there, and the routers read those columns alone (a norm scales them all alike, which keeps the order of the logits).
"""
import os

import torch

MARKERS = 3
MARK = 2.0
MARGIN = 0.1         # least distance between the last chosen logit and the first left out, markers taken as +-1


def _left(heads, kv_heads, dim, vdim, scale, rot_dims=None, base=10000.0, scaling=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot_dims:
        m["rot"] = dict(dims=rot_dims, base=base)
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return m


def _parallel(left, right, ls, rs, mlp, **kw):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp, **kw}


def _right(heads, dim, vdim, decay):
    return dict(heads=heads, dim=dim, vdim=vdim, decay=decay)


def _gla(heads, dim, vdim, tau, mlp, **kw):
    return {"type": "gla", "mixer": dict(heads=heads, dim=dim, vdim=vdim, tau=tau), "mlp": mlp, **kw}


def _moe(ff, experts, top, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


_A0 = _parallel(_left(6, 2, 16, 24, 0.3, rot_dims=8, base=50.0, scaling=(8.0, 1.0, 4.0, 64)),
                _right(3, 8, 16, [0.9, 0.97, 0.995]), 0.7, 0.4, _moe(24, 5, 2, shared=40))
_A1 = _gla(2, 16, 24, 8.0, _moe(32, 4, 2, shared=16))
_B1 = _parallel(_left(4, 4, 16, 16, 0.25, rot_dims=16, base=10000.0), _right(1, 16, 16, [1.0]), 1.0, 1.0, _moe(24, 3, 1))

MODELS = {
    "A": dict(
        config={"architecture": "Lilalorn", "vocab": 331, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
                "logit_scale": 0.4, "layers": [
                    _A0, _A1, dict(_A0, weights_of=0),
                    _parallel(_left(4, 1, 32, 8, 0.2, rot_dims=32, base=300.0), _right(2, 16, 8, [0.5, 0.999]), 0.5, 0.8, None),
                    dict(_A1, weights_of=1)]},
        seed=21, linear_std=0.1, norm_std=0.1, page_size=16, decay_rank=8),
    "B": dict(
        config={"architecture": "Lilalorn", "vocab": 257, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
                "logit_scale": 1.0, "layers": [
                    _gla(1, 16, 16, 1.0, _moe(24, 3, 1, shared=24)),
                    _B1,
                    _parallel(_left(2, 2, 32, 32, 0.18, rot_dims=32, base=1000.0), _right(2, 8, 8, [0.05, 1.0]), 1.0, 1.0,
                              _moe(16, 2, 2, shared=8)),
                    dict(_B1, weights_of=1)]},
        seed=22, linear_std=0.12, norm_std=0.2, page_size=8, decay_rank=12),
    "O": dict(
        config={"architecture": "Lilalorn", "vocab": 131, "width": 50, "norm": {"eps": 1e-5}, "residual_mult": 0.8,
                "logit_scale": 1.5, "layers": [
                    _parallel(_left(3, 1, 12, 20, 0.3, rot_dims=6, base=100.0), _right(2, 10, 6, [0.8, 0.99]), 0.9, 0.6,
                              _moe(18, 4, 2, shared=10)),
                    _gla(3, 10, 14, 4.0, _moe(18, 3, 2))]},
        seed=23, linear_std=0.1, norm_std=0.1, page_size=8, decay_rank=5),
    "G": dict(
        config={"architecture": "Lilalorn", "vocab": 150, "width": 48, "norm": {"eps": 1e-5}, "residual_mult": 0.9,
                "logit_scale": 2.0, "layers": [_gla(2, 8, 16, 2.0, None), _gla(3, 16, 8, 32.0, _moe(16, 3, 2, shared=8)),
                                               dict(_gla(2, 8, 16, 2.0, None), weights_of=0)]},
        seed=25, linear_std=0.15, norm_std=0.1, page_size=8, decay_rank=4),
    "R": dict(
        config={"architecture": "Lilalorn", "vocab": 409, "width": 512, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
                "logit_scale": 0.25, "layers": [
                    _parallel(_left(8, 2, 64, 128, 0.125, rot_dims=64, base=500000.0, scaling=(8.0, 1.0, 4.0, 8192)),
                              _right(4, 64, 128, [0.97, 0.99, 0.995, 0.999]), 0.7, 0.5, _moe(128, 6, 2, shared=256)),
                    _gla(2, 128, 256, 12.0, _moe(128, 6, 2, shared=256)),
                    _gla(1, 192, 64, 20.0, None)]},
        seed=24, linear_std=0.04, norm_std=0.1, page_size=64, decay_rank=24),
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
    ids = torch.arange(c["vocab"])
    for b, col in enumerate(cols):
        W["embed"][:, col] = (((ids >> b) & 1).float() * 2 - 1) * MARK
    g = torch.Generator().manual_seed(t["seed"])
    for name_, w in W.items():
        if name_.endswith((".o", ".down")):                 # nothing but the embedding writes to the marker columns
            w[cols, :] = 0
        if name_.endswith(".a2.b"):                         # decays from about 0.5 to nearly 1 (with tau 1; nearer 1 with more).
            # Much stronger ones leave a token's result to q . k of that token alone, whose sign bfloat16 does not keep
            # where it is near zero, and the heads' norm then turns a small difference into a large one
            w.copy_((torch.randn(w.shape, generator=g) + 1.5).to(w.dtype))
        if name_.endswith((".a1", ".a2")) and w.dim() == 2:
            w.mul_(4.0)
    # A token's own share of its state's answer is (q . k) v.  Where that product is near zero its sign is left to
    # bfloat16's rounding, and the heads' norm, which divides by the answer's size, makes a large difference of a
    # small one (most of all in a sequence's first tokens, whose answer has few shares).  The tests' keys therefore
    # lean towards their queries: the own share is clearly positive, and the tolerances can stay tight.
    for name_ in list(W):
        if name_.endswith((".mix.k", ".mix.right.k")):
            W[name_] = (W[name_[:-1] + "q"].float() + 0.5 * W[name_].float()).to(torch.bfloat16)
    for i, layer in enumerate(c["layers"]):
        rank = t.get("decay_rank")
        if layer["type"] == "gla" and layer.get("weights_of") is None and rank and W[f"l{i}.mix.a1"].shape[0] != rank:
            # the rank of the decay's projection is the tensors' own: any will do
            W[f"l{i}.mix.a1"] = (torch.randn(rank, width, generator=g) * 4 * t["linear_std"]).to(torch.bfloat16)
            W[f"l{i}.mix.a2"] = (torch.randn(W[f"l{i}.mix.a2"].shape[0], rank, generator=g) * 4 * t["linear_std"]).to(torch.bfloat16)
        ml = layer.get("mlp")
        if not ml or layer.get("weights_of") is not None:
            continue
        W[f"l{i}.norm2"][cols] = 1.0
        top, experts = ml["router"]["top"], ml["router"]["experts"]
        pats = torch.tensor([[1.0 if (p >> b) & 1 else -1.0 for b in range(MARKERS)] for p in range(1 << MARKERS)])
        for _ in range(20000):            # until every pattern's choice is clear by MARGIN
            rw = (torch.randn(experts, MARKERS, generator=g) * 0.5).to(torch.bfloat16).float()
            z = (pats @ rw.T).sort(dim=-1, descending=True).values
            if top == experts or float((z[:, top - 1] - z[:, top]).min()) >= MARGIN:
                break
        else:
            raise RuntimeError("no decisive router found")
        r = torch.zeros_like(W[f"l{i}.mlp.router"], dtype=torch.float32)
        r[:, cols] = rw
        W[f"l{i}.mlp.router"] = r.to(torch.bfloat16)
    save_file({k: v.contiguous() for k, v in W.items()}, path)
    return model_dir


def router_margin(model_dir, tokens):
    """The least distance, over a sequence's tokens and the model's routers, between the last chosen expert's
    logit and the first one left out, as a fraction of the largest logit of that token (float64, plain)."""
    import plain_lilalorn as plain
    pm = plain.PlainLilalorn(model_dir, torch.float64)
    least = float("inf")
    x = pm.W["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(pm.c["layers"]):
        ml = layer.get("mlp")
        if not ml or ml["router"]["top"] == ml["router"]["experts"]:
            continue
        p = f"l{pm.tensors_of(i)}"
        # the routers read the marker columns alone, which no branch changes: the embedding's rows will do for the stream
        z = pm.router_logits(p + ".mlp", plain.rms_norm(x, pm.eps, pm.W[p + ".norm2"]))
        top = ml["router"]["top"]
        val, _ = z.topk(top + 1, dim=-1)
        least = min(least, float(((val[:, top - 1] - val[:, top]) / z.abs().max(dim=-1).values).min()))
    return least
