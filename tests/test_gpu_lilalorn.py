"""Lilalorn on the GPU against the plain implementation (tests/plain_lilalorn.py): each mechanism's kernel
alone, then whole models under every way of cutting the work, in float32 and bfloat16."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import harness
import plain_lilalorn as plain
from lilalorn_models import MODELS, make_model, router_margin

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("lilalorn")
    made = {}

    def get(name):
        if name not in made:
            made[name] = make_model(str(root / name), name)
        return made[name]
    return get


# ---- the decaying state ----------------------------------------------------------------------------------
def _scan_inputs(T, H, dk, dv, dt, seed, per_token):
    g = torch.Generator().manual_seed(seed)
    packed = (torch.randn(T, 2 * H * dk + H * dv + 5, generator=g) * 0.5).to(dt)       # q | k | v | something else
    q, k, v = packed[:, :H * dk], packed[:, H * dk:2 * H * dk], packed[:, 2 * H * dk:2 * H * dk + H * dv]
    z = torch.randn(T, H * dk, generator=g) * 3 if per_token else None
    bias = torch.randn(H * dk, generator=g) if per_token else None
    decay = None if per_token else torch.rand(H, generator=g) * 0.2 + 0.8
    return packed, q, k, v, z, bias, decay


def _decays(T, H, dk, z, bias, decay, tau):
    if z is not None:
        return torch.sigmoid(z.double() + bias.double()).pow(1.0 / tau).view(T, H, dk)
    return decay.double()[None, :, None].expand(T, H, dk)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [0, 16])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("H,dk,dv", [(2, 16, 24), (3, 10, 6), (1, 192, 64), (2, 128, 256), (1, 7, 70), (1, 256, 8)])
def test_state_walk_of_unequal_requests_in_portions(H, dk, dv, per_token, chunk, dtype, monkeypatch):
    """Three requests of unequal length in one batch, in slots that are not in order, cut into portions of several
    sizes down to one token: every portion starts from the state the one before left in the slot.  With `chunk`
    the long portions are walked in chunks of 16 tokens side by side (a last chunk of one token, a chunked portion
    beside single tokens), the short ones in one piece."""
    from xinfer_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_CHUNK", chunk)
    dt, tau = TD[dtype], 4.0
    lens = [37, 5, 70]
    cuts = {0: [2, 33, 1, 1], 1: [5], 2: [1, 1, 2, 64, 2]}
    slots = [3, 0, 2]
    data = [_scan_inputs(n, H, dk, dv, dt, 10 * i + H, per_token) for i, n in enumerate(lens)]
    want = []
    for n, (_, q, k, v, z, _, _) in zip(lens, data):           # the bias and the heads' decays are the layer's: the first's
        o, _ = plain.decaying_state(q.double().view(n, H, dk) * 0.5, k.double().view(n, H, dk) * 0.25, v.double().view(n, H, dv),
                                    _decays(n, H, dk, z, data[0][5], data[0][6], tau))
        want.append(o)
    state = torch.full((5, H, dk, dv), 7.0, device=DEV)          # what another request left
    state[slots] = 0
    got = [[] for _ in lens]
    at = [0] * len(lens)
    for step in range(5):
        rows, cu, who = [], [0], []
        for b in range(len(lens)):
            if step < len(cuts[b]):
                n = cuts[b][step]
                rows.append((b, at[b], n))
                cu.append(cu[-1] + n)
                who.append(b)
                at[b] += n
        packed = torch.cat([data[b][0][a:a + n] for b, a, n in rows]).to(DEV)
        q, k, v = packed[:, :H * dk], packed[:, H * dk:2 * H * dk], packed[:, 2 * H * dk:2 * H * dk + H * dv]
        zz = torch.cat([data[b][4][a:a + n] for b, a, n in rows]).to(DEV) if per_token else None
        o = kernels.linear_scan(q, k, v, state, torch.tensor([slots[b] for b in who], device=DEV),
                                torch.tensor(cu, dtype=torch.int32, device=DEV), H, dk, dv, z=zz, tau=tau,
                                z_bias=data[0][5].to(DEV) if per_token else None,
                                head_decay=None if per_token else data[0][6].to(DEV), q_scale=0.5, k_scale=0.25,
                                q_lens=[n for _, _, n in rows] if chunk else None, plan_cache={} if step % 2 else None)
        for i, (b, a, n) in enumerate(rows):
            got[b].append(o[cu[i]:cu[i + 1]].cpu())
    assert torch.all(state[1] == 7.0) and torch.all(state[4] == 7.0)        # other slots are left alone
    for b, n in enumerate(lens):
        g = torch.cat(got[b]).double()
        assert g.shape == want[b].shape
        assert (g - want[b]).abs().max() < 2e-5 * want[b].abs().max(), (b, float((g - want[b]).abs().max()))


def test_the_cutting_of_long_portions():
    from xinfer_amd import kernels
    whole, long, chunks = kernels.scan_chunk_plan([1, 130, 64, 128, 300, 127], 64)
    assert whole == [0, 2, 5] and long == [(1, 0, 3), (3, 3, 2), (4, 5, 5)]
    assert chunks == [(0, 64), (64, 64), (128, 2), (0, 64), (64, 64), (0, 64), (64, 64), (128, 64), (192, 64), (256, 44)]
    assert kernels.scan_chunk_plan([500, 3], 0) == ([0, 1], [], [])
    _, long, chunks = kernels.scan_chunk_plan([100_000], 64)           # no more chunks than their states have room for
    assert len(chunks) <= kernels.SCAN_CHUNKS_MOST and sum(n for _, n in chunks) == 100_000


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("decay,far", [(1.0, 599), (0.999, 300), (0.9, 40)])
def test_state_keeps_a_far_key(decay, far, dtype):
    """One key far back is made to stand out (its k and the last q are scaled up along one direction): the last
    token's result is that token's value times decay^distance, which a lost or reset state would not give;
    the prompt is cut at a place of its own and decoded one by one at the end."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    T, H, dk, dv = 600, 2, 32, 40
    g = torch.Generator().manual_seed(far)
    q = (torch.randn(T, H * dk, generator=g) * 0.1).to(dt)
    k = (torch.randn(T, H * dk, generator=g) * 0.1).to(dt)
    v = torch.randn(T, H * dv, generator=g).to(dt)
    at = T - 1 - far
    k[:, 3] = 0                       # head 0's channel 3 belongs to the planted key alone
    k[at, :dk] = 0
    k[at, 3] = 30.0
    q[T - 1, 3] = 30.0
    want, _ = plain.decaying_state(q.double().view(T, H, dk), k.double().view(T, H, dk), v.double().view(T, H, dv),
                                   torch.full((T, H, dk), decay, dtype=torch.float64))
    expected_share = 900.0 * decay ** far * v.double().view(T, H, dv)[at, 0]
    assert (want[T - 1, 0] - expected_share).abs().max() < 0.1 * expected_share.abs().max()      # the planted key dominates
    state = torch.zeros(1, H, dk, dv, device=DEV)
    slot = torch.zeros(1, dtype=torch.int64, device=DEV)
    outs = []
    for a, b in [(0, 257), (257, T - 5)] + [(t, t + 1) for t in range(T - 5, T)]:
        cu = torch.tensor([0, b - a], dtype=torch.int32, device=DEV)
        outs.append(kernels.linear_scan(q[a:b].to(DEV), k[a:b].to(DEV), v[a:b].to(DEV), state, slot, cu, H, dk, dv,
                                        head_decay=torch.full((H,), decay, device=DEV), q_lens=[b - a]).cpu())
    got = torch.cat(outs).double()
    assert (got - want).abs().max() < 3e-5 * want.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_norm_and_gate(dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(5)
    for T, H, dv, weighted in ((9, 3, 24, True), (4, 2, 70, False), (130, 1, 256, True)):
        o = torch.randn(T, H, dv, generator=g) * 3
        packed = torch.randn(T, H * dv + 11, generator=g).to(dt)
        gate = packed[:, 11:]
        w = 1 + 0.3 * torch.randn(dv, generator=g) if weighted else None
        want = plain.rms_norm(o.double(), 1e-5, None if w is None else w.double()).reshape(T, H * dv) * plain.silu(gate.double())
        got = kernels.head_norm_gate(o.to(DEV), None if w is None else w.to(DEV), 1e-5, packed.to(DEV)[:, 11:], dt)
        tol = 1e-5 if dt == torch.float32 else 1e-2
        assert got.dtype == dt and (got.cpu().double() - want).abs().max() < tol * want.abs().max()


# ---- rotation, cache write and attention with a planted key -------------------------------------------------
def _pools(L, G, d, dv, page, dtype, grouped, seed=0):
    n_pages = -(-L // page)
    order = list(range(n_pages + 3))
    random.Random(seed).shuffle(order)
    table = torch.tensor([order[:n_pages]], dtype=torch.int32)
    k_pool = torch.zeros(n_pages + 3, G, page, d, dtype=dtype)
    v_pool = torch.zeros((n_pages + 3, G, page // 8, dv, 8) if grouped else (n_pages + 3, G, page, dv), dtype=dtype)
    slots = torch.tensor([order[p // page] * page + p % page for p in range(L)], dtype=torch.int64)
    return k_pool, v_pool, table, slots


ROTS = [dict(dims=8, base=50.0, scaling=dict(factor=8.0, low=1.0, high=4.0, original=64)), dict(dims=16, base=10000.0),
        dict(dims=6, base=100.0)]


def test_frequency_scaling_has_all_three_bands():
    sc = ROTS[0]
    plain_f = plain.rotary_frequencies(dict(dims=sc["dims"], base=sc["base"]))
    scaled = plain.rotary_frequencies(sc)
    ratio = (scaled / plain_f).tolist()
    assert ratio[0] == 1.0 and abs(ratio[-1] - 1 / 8) < 1e-12 and any(1 / 8 + 1e-3 < r < 1 - 1e-3 for r in ratio)
    from xinfer_amd.parts.rope import scaled_inv_freq
    inv, m = scaled_inv_freq(sc["base"], sc["dims"], dict(kind="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original=64))
    assert m == 1.0 and np.allclose(inv, scaled.numpy(), rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,rot", [(6, 2, 16, 24, ROTS[0]), (4, 4, 16, 16, ROTS[1]), (3, 1, 12, 20, ROTS[2]), (2, 1, 32, 8, ROTS[1])])
def test_rotation_and_attention_with_a_planted_key(H, G, d, dv, rot, dtype):
    """q and k turned by position and written through pages (a portion, a second one that starts inside a page,
    then single tokens), then attention over them: one key far back, at a page's border, is made to stand out
    through the dims that do not turn (or through the score's own maximum where all turn)."""
    from xinfer_amd import kernels
    from xinfer_amd.config.spec import PartSpec
    from xinfer_amd.parts.rope import RotaryEmbedding
    dt = TD[dtype]
    grouped = dt == torch.bfloat16
    L, page, scale = 150, 16, 0.3
    g = torch.Generator().manual_seed(H * d)
    qkv = (torch.randn(L, H * d + G * d + G * dv, generator=g) * 0.7).to(dt)
    far = 47 if rot["dims"] < d else 48          # the last key of a page, the first of the next
    if rot["dims"] < d:
        qkv[L - 1, d - 1] = 9.0                      # head 0's last dim, which does not turn
        qkv[far, H * d + d - 1] = 9.0
    q = qkv[:, :H * d].double().view(L, H, d)
    k = qkv[:, H * d:H * d + G * d].double().view(L, G, d)
    v = qkv[:, H * d + G * d:].double().view(L, G, dv)
    pos = torch.arange(L)
    want = plain.softmax_attention(plain.rotate(q, rot, pos), plain.rotate(k, rot, pos), v, scale).reshape(L, H * dv)
    if rot["dims"] < d:
        assert (want[L - 1, :dv] - v[far, 0]).abs().max() < 0.05 * v[far, 0].abs().max()
    enc = RotaryEmbedding(PartSpec("rope", dict(head_dim=d, rotary_dim=rot["dims"], theta=rot["base"], max_positions=256,
                                                scaling=None if "scaling" not in rot else dict(
                                                    kind="llama3", factor=rot["scaling"]["factor"], low_freq_factor=rot["scaling"]["low"],
                                                    high_freq_factor=rot["scaling"]["high"], original=rot["scaling"]["original"]))), dt)
    enc.load(None, "", DEV)
    k_pool, v_pool, table, slots = (t.to(DEV) for t in _pools(L, G, d, dv, page, dt, grouped, seed=d))
    outs = []
    for a, b in [(0, 41), (41, L - 4)] + [(t, t + 1) for t in range(L - 4, L)]:
        positions = torch.arange(a, b, dtype=torch.int32, device=DEV)
        qr = kernels.qkv_rows(qkv[a:b].to(DEV), None, None, 0.0, slots[a:b], k_pool, v_pool, H, G, d, dv, v_grouped=grouped,
                              cos=enc.cos, sin=enc.sin, rotary_dim=rot["dims"], positions=positions)
        outs.append(kernels.attention_generic(qr, k_pool, v_pool, table, torch.zeros(b - a, dtype=torch.int32, device=DEV),
                                              positions, scale, v_grouped=grouped).cpu())
    got = torch.cat(outs).double()
    tol = 2e-5 if dt == torch.float32 else 2e-2
    assert (got - want).abs().max() < tol * want.abs().max()


# ---- the feed-forward's parts --------------------------------------------------------------------------------
@pytest.mark.parametrize("E,top,H", [(5, 2, 96), (3, 1, 100), (16, 4, 320), (7, 7, 64)])
def test_router_scores_over_all_experts_and_the_shared_gate(E, top, H):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(E)
    x = torch.randn(33, H, generator=g)
    r = torch.randn(E + 1, H, generator=g) * 0.3                 # the last row opens the shared branch
    idx, wt = plain.router_weights(x.double() @ r[:E].double().T, top)
    gi, gw, extra = kernels.moe_route(x.to(DEV), r.to(DEV), None, top, all_scores=True, extra_rows=1)
    assert torch.equal(gi.cpu().long(), idx)
    assert (gw.cpu().double() - wt).abs().max() < 1e-6
    assert (extra.cpu().double()[:, 0] - x.double() @ r[E].double()).abs().max() < 1e-5
    # the two ways of weighing agree where the mathematics says so, and differ in their bits' path only
    ci, cw = kernels.moe_route(x.to(DEV), r[:E].contiguous().to(DEV), None, top)
    assert torch.equal(ci, gi) and (cw - gw).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,H,F,T", [(5, 2, 96, 48, 19), (3, 1, 100, 24, 5), (6, 2, 512, 128, 300), (4, 4, 64, 200, 1)])
def test_experts_without_a_gate(E, top, H, F, T, dtype):
    """down(relu(up x)^2), a pair at a time, grouped on the matrix cores and through the library, with a shared
    expert opened by a sigmoid."""
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(F)
    x = torch.randn(T, H, generator=g).to(dt)
    r = torch.randn(E + 1, H, generator=g) * 0.3
    up = (torch.randn(E, F, H, generator=g) * 0.1).to(dt)
    down = (torch.randn(E, H, F, generator=g) * 0.1).to(dt)
    idx, wt = plain.router_weights(x.double() @ r[:E].double().T, top)
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            want[t] += wt[t, j] * plain.expert(x[t].double(), up[e].double(), down[e].double())
    gi, gw, extra = kernels.moe_route(x.to(DEV), r.to(DEV), None, top, all_scores=True, extra_rows=1)
    tol = 1e-5 if dt == torch.float32 else 2e-2
    got = kernels.moe_experts(x.to(DEV), up.to(DEV), down.to(DEV), gi, gw, "relu2", grouped=False, gated=False)
    assert got.dtype == torch.float32 and (got.cpu().double() - want).abs().max() < tol * want.abs().max()
    if dt == torch.bfloat16 and H % 8 == 0 and F % 8 == 0:
        for rows in (32, 64, 128):
            grp = kernels.moe_experts(x.to(DEV), up.to(DEV), down.to(DEV), gi, gw, "relu2", grouped=True, tile_rows=rows, gated=False)
            assert (grp.cpu().double() - want).abs().max() < tol * want.abs().max()
        lib = kernels.moe_experts_library(x.to(DEV), up.to(DEV), down.to(DEV), gi, gw, "relu2", gated=False)
        assert (lib.cpu().double() - want).abs().max() < tol * want.abs().max()
    # the shared branch: out += sigmoid(gate) * y
    y = torch.randn(T, H, generator=g).to(dt)
    kernels.gated_add_(got, y.to(DEV), extra[:, 0])
    want2 = want + torch.sigmoid(x.double() @ r[E].double())[:, None] * y.double()
    assert (got.cpu().double() - want2).abs().max() < tol * want2.abs().max()


def test_a_factor_on_the_branch_that_a_norm_adds():
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(2)
    for width in (96, 50, 1000):
        x = torch.randn(7, width, generator=g)
        w = 1 + 0.2 * torch.randn(width, generator=g)
        for y in (torch.randn(7, width, generator=g), torch.randn(7, width, generator=g).to(torch.bfloat16),
                  torch.randn(3, 7, width, generator=g)):
            resid = x.to(DEV).clone()
            out = kernels.add_rmsnorm(resid, y.to(DEV), w.to(DEV), 1e-5, torch.float32, y_scale=0.7)
            s = x.double() + 0.7 * (y.double() if y.dim() == 2 else y.double().sum(0))
            assert (resid.cpu().double() - s).abs().max() < 1e-5
            assert (out.cpu().double() - plain.rms_norm(s, 1e-5, w.double())).abs().max() < 1e-5
            one = x.to(DEV).clone()
            kernels.add_rmsnorm(one, y.to(DEV), w.to(DEV), 1e-5, torch.float32)                 # a factor of 1 is the plain sum
            ref = x.clone()
            for part in (y.float().unsqueeze(0) if y.dim() == 2 else y):
                ref += part
            assert torch.equal(one.cpu(), ref)
        # rows only: the stream is left alone
        resid = x.to(DEV).clone()
        rows = torch.tensor([5, 0], dtype=torch.int32, device=DEV)
        out = kernels.add_rmsnorm(resid, y[0].contiguous().to(DEV), w.to(DEV), 1e-5, torch.float32, rows=rows, y_scale=0.5)
        assert torch.equal(resid.cpu(), x)
        s = (x.double() + 0.5 * y[0].double())[[5, 0]]
        assert (out.cpu().double() - plain.rms_norm(s, 1e-5, w.double())).abs().max() < 1e-5
    a = kernels.scaled_sum(None, torch.ones(2, 3, device=DEV, dtype=torch.bfloat16), 0.5)
    kernels.scaled_sum(a, torch.ones(2, 2, 3, device=DEV), 2.0)
    assert torch.equal(a.cpu(), torch.full((2, 3), 4.5))
    assert torch.equal(kernels.act_(torch.tensor([-1.0, 0.5, 3.0], device=DEV), "relu2").cpu(), torch.tensor([0.0, 0.25, 9.0]))
    assert torch.equal(kernels.scale_(torch.tensor([2.0, -4.0], device=DEV), 0.25).cpu(), torch.tensor([0.5, -1.0]))


# ---- whole models ----------------------------------------------------------------------------------------------
LENGTHS = {"A": [1, 2, 12, 13, 33, 77, 130], "B": [3, 9, 10, 18, 64, 101], "O": [1, 7, 8, 40, 75], "G": [2, 1, 30, 140],
           "R": [5, 101, 330, 64, 301]}


def _requests(name):
    rng = random.Random(700 + ord(name))
    vocab = MODELS[name]["config"]["vocab"]
    return {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}
_model_cache = {}


def _plain_logits(name, model_dir):
    if name not in _plain_cache:
        pm = plain.PlainLilalorn(model_dir, torch.float64)
        _plain_cache[name] = {rid: pm.logits(toks).float() for rid, toks in _requests(name).items()}
    return _plain_cache[name]


def _model(name, dtype, model_dir):
    from xinfer_amd.engine import load_model
    if (name, dtype) not in _model_cache:
        _model_cache[(name, dtype)] = load_model(model_dir, dtype, DEV)
    return _model_cache[(name, dtype)]


def _run(name, dtype, dirs, steps, what, **kw):
    from xinfer_amd.engine import ModelRunner
    page = MODELS[name]["page_size"]
    need = harness.tokens_needed(steps, page)
    model = _model(name, dtype, dirs(name))
    runner = ModelRunner(model, page_size=page, num_pages=max(1, need // page), max_requests=4, **kw)     # exactly enough pages
    got = harness.replay(runner, steps)
    for g in range(len(runner.cache.groups)):
        assert runner.cache.free_pages(g) == max(1, need // page)
    rel = harness.compare(got, _plain_logits(name, dirs(name)), harness.TOL[dtype], f"{name}/{dtype}/{what}")
    print(f"{name}/{dtype}/{what}: worst error {rel:.2e} of the largest logit")
    return got, runner


@pytest.mark.parametrize("name", list(MODELS))
def test_the_models_are_what_they_are_meant_to_be(name, dirs):
    from xinfer_amd.engine import load_model
    for toks in _requests(name).values():
        assert router_margin(dirs(name), toks) > 0.03
    model = _model(name, "float32", dirs(name))
    layers = MODELS[name]["config"]["layers"]
    assert len(model.spec.schedule) == len(layers)
    assert len(model.blocks) == sum(1 for l in layers if l.get("weights_of") is None)
    assert len(model.state_needs) == len(layers)                               # every run keeps a state of its own
    assert len(model.kv_needs) == sum(1 for l in layers if l["type"] == "parallel")
    assert model.graph_safe


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_whole(name, dtype, dirs):
    got, _ = _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole")
    assert len(got) == sum(LENGTHS[name])


def test_the_stream_after_every_layer(dirs):
    """float32, one request: the residual stream after every run of a layer against the plain one."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    name = "A"
    model = _model(name, "float32", dirs(name))
    toks = _requests(name)["r4"]
    want = plain.PlainLilalorn(dirs(name), torch.float64).stream(toks)[1:]
    seen = []
    kept = [(b, b.forward) for b in model.blocks]
    try:
        for blk, orig in kept:
            def fwd(stream, ctx, c, _o=orig, **kw):
                s = _o(stream, ctx, c, **kw)
                p = s.pending.float() if s.pending.dim() == 2 else s.pending.float().sum(0)
                seen.append((s.resid + s.pending_scale * p).cpu().double())
                return s
            blk.forward = fwd
        runner = ModelRunner(model, page_size=16, num_pages=4, max_requests=1, use_graphs=False)
        runner.add_request(0)
        runner.step([StepEntry(0, toks, [])])
    finally:
        for blk, orig in kept:
            blk.forward = orig
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        assert (a - b).abs().max() < 1e-5 * b.abs().max(), f"the stream after layer run {i} differs"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_prefill_against_decoding_one_by_one(name, dtype, dirs):
    _run(name, dtype, dirs, harness.trace_tail_one_by_one(_requests(name), tail=40), "tail")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_portions(name, dtype, dirs):
    _run(name, dtype, dirs, harness.trace_portions(_requests(name)), "portions")
    _run(name, dtype, dirs, harness.trace_portions(_requests(name), sizes=(2, 2, 3, 40, 2, 5)), "small portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, dirs):
    """More requests than state slots, one after the other in the same slots and pages: a request that starts
    finds no state of the one before."""
    for seed in (1, 2):
        _run(name, dtype, dirs, harness.trace_mixed(_requests(name), seed, max_live=3), f"mixed {seed}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "O"])
def test_short_chunks_of_the_states_walk(name, dtype, dirs, monkeypatch):
    """Portions from 32 tokens on are walked in chunks of 16: whole prompts, portions and mixed batches again."""
    from xinfer_amd import kernels
    monkeypatch.setattr(kernels, "SCAN_CHUNK", 16)
    _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole, chunks of 16")
    _run(name, dtype, dirs, harness.trace_portions(_requests(name), sizes=(33, 2, 47, 32, 5)), "portions, chunks of 16")
    _run(name, dtype, dirs, harness.trace_mixed(_requests(name), 3, max_live=3, sizes=(40, 2, 35, 64)), "mixed, chunks of 16")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_unequal_requests_decoding_together(name, dtype, dirs):
    reqs = {k: v for k, v in _requests(name).items() if len(v) > 8}
    reqs = dict(list(reqs.items())[:4])
    _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode", use_graphs=False)
    got, runner = _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode, graphs", graph_after=1)
    assert runner.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype, dirs):
    """Three tokens of prompt, then 250 one by one: the states and the pages grow token by token over many pages."""
    name = "A"
    toks = harness.random_prompt(random.Random(9), 253, MODELS[name]["config"]["vocab"])
    from xinfer_amd.engine import ModelRunner
    ref = {"a": plain.PlainLilalorn(dirs(name), torch.float64).logits(toks).float()}
    steps = harness.trace_tail_one_by_one({"a": toks}, tail=250)
    runner = ModelRunner(_model(name, dtype, dirs(name)), page_size=16, num_pages=16, max_requests=2, graph_after=2)
    got = harness.replay(runner, steps)
    assert runner.graph_replays > 200
    harness.compare(got, ref, harness.TOL[dtype], f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_through_the_engine(dtype, dirs):
    """The framework's own entry point and scheduler: five prompts, three at a time, prompts cut into
    portions of 16 tokens, greedy tokens against the plain implementation."""
    from xinfer_amd import Engine, EngineConfig, SamplingParams
    name = "A"
    rng = random.Random(3)
    vocab = MODELS[name]["config"]["vocab"]
    prompts = [harness.random_prompt(rng, n, vocab) for n in (5, 40, 17, 33, 2)]
    eng = Engine(EngineConfig(weight_path=dirs(name), page_size=16, num_pages=24, max_num_seqs=3, prefill_chunk_size=16,
                              max_model_len=128, seed=1), dtype)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    if dtype == "f32":        # a model without pages, the engine planning its own (token counts alone)
        g_eng = Engine(EngineConfig(weight_path=dirs("G"), page_size=8, max_num_seqs=2, prefill_chunk_size=16, max_model_len=64,
                                    seed=1), dtype)
        g_prompts = [[5, 9, 77, 3], list(range(40, 75))]
        g_outs = g_eng.generate(g_prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
        g_plain = plain.PlainLilalorn(dirs("G"), torch.float64)
        assert [o.token_ids for o in g_outs] == [g_plain.greedy(p, 10) for p in g_prompts]
    pm = plain.PlainLilalorn(dirs(name), torch.float64)
    for p, o in zip(prompts, outs):
        assert o.prompt_length == len(p) and o.decoded_length == 24
        if dtype == "f32":
            assert o.token_ids == pm.greedy(p, 24)
        else:
            ids = list(p)
            for t in o.token_ids:
                lg = pm.logits(ids)[-1]
                assert float(lg.max() - lg[t]) <= 2 * harness.TOL["bfloat16"] * float(lg.abs().max())
                ids.append(t)
    assert eng.runner.cache.live_requests() == 0


def test_command_line_runs_the_model(dirs, capsys):
    from xinfer_amd import cli
    rc = cli.main(["--w", dirs("A"), "--prompt-ids", "1,2,3,4,5,6,7,8,9", "--max-tokens", "4", "--max-model-len", "256",
                   "--temperature", "0", "--ignore-eos", "--page-size", "16", "--max-num-seqs", "4", "--dtype", "bf16"])
    assert rc == 0 and "Decoded tokens: 4 in" in capsys.readouterr().out
    rc = cli.main(["--w", dirs("B"), "--prompt-ids", "1,2,3|4,5,6,7", "--max-tokens", "5", "--max-model-len", "64",
                   "--temperature", "0", "--ignore-eos", "--page-size", "8", "--num-pages", "16", "--dtype", "f32"])
    assert rc == 0 and "Decoded tokens: 10 in" in capsys.readouterr().out


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dtype, dirs, tmp_path):
    name = "B"
    vocab = MODELS[name]["config"]["vocab"]
    reqs = {f"r{i}": harness.random_prompt(random.Random(60 + i), n, vocab) for i, n in enumerate([33, 70, 5, 64, 100, 9])}
    steps = harness.trace_mixed(reqs, 4)
    need = harness.tokens_needed(steps, 64)
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, os.path.join(REPO, "bin", "trace_run"), "--model", dirs(name), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(need)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:
        proc.stdin.write(json.dumps(st) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {st['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0
    pm = plain.PlainLilalorn(dirs(name), torch.float64)
    ref = {rid: pm.logits(t).float() for rid, t in reqs.items()}
    got, fed = {}, {rid: 0 for rid in reqs}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        arr = np.fromfile(out / f"{st['step']}.f32", dtype="<f4").reshape(wanted, vocab)
        row = 0
        for e in st["entries"]:
            for w in e["want"]:
                got[(e["id"], fed[e["id"]] + w)] = torch.from_numpy(arr[row].copy())
                row += 1
            fed[e["id"]] += len(e["tokens"])
    assert len(got) == sum(len(t) for t in reqs.values())
    harness.compare(got, ref, harness.TOL[dtype], f"trace_run {dtype}")


def test_decode_graph_replays_equal_launches(dirs):
    """float32: steps replayed from a recorded graph give the bits of the same steps launched one by one (the
    states are advanced once a step, in the step that records too)."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    name = "A"
    model = _model(name, "float32", dirs(name))
    vocab, page = MODELS[name]["config"]["vocab"], MODELS[name]["page_size"]
    rng = random.Random(21)
    prompts = {i: harness.random_prompt(rng, rng.randrange(3, 50), vocab) for i in range(4)}
    feed = {i: harness.random_prompt(rng, 30, vocab) for i in prompts}

    def run(use_graphs):
        runner = ModelRunner(model, page, 24, 4, use_graphs=use_graphs, graph_after=1)
        out = []
        for i in prompts:
            runner.add_request(i)
            runner.step([StepEntry(i, prompts[i], [])])
        for step in range(30):
            out.append(runner.step([StepEntry(i, [feed[i][step]], [0]) for i in prompts]).cpu())
        return out, runner
    want, _ = run(False)
    got, r1 = run(True)
    assert r1.graph_replays >= 25
    for k, (a, b) in enumerate(zip(want, got)):
        assert torch.equal(a, b), f"step {k} differs between graph and launches"
