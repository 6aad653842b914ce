"""Mufenex on the GPU against the plain implementation (tests/plain_mufenex.py): each mechanism's
kernel alone, then whole models under every way of cutting the work, in float32 and bfloat16."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import harness
import plain_mufenex as plain
from mufenex_models import MODELS, make_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("mufenex")
    made = {}

    def get(name):
        if name not in made:
            made[name] = make_model(str(root / name), name)
        return made[name]
    return get


# ---- mechanisms alone -------------------------------------------------------------------------------
def test_embedding_with_sinusoidal_positions():
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(0)
    for width, scale in ((96, 0.7), (101, 1.0)):
        table = torch.randn(50, width, generator=g).to(torch.bfloat16)
        ids = torch.randint(0, 50, (300,), generator=g)
        first = 4000
        freq = torch.tensor(10000.0) ** (-2.0 * torch.arange((width + 1) // 2, dtype=torch.float32) / width)
        pos = torch.arange(first, first + 300, dtype=torch.int32)
        want = table.float()[ids] * scale + plain.sinusoid_positions(300, width, torch.float32, first=first)
        for dt in (torch.float32, torch.bfloat16):
            out, rows = kernels.embed_sinusoid(table.to(dt).to(DEV), ids.int().to(DEV), pos.to(DEV), freq.to(DEV), scale,
                                               None if dt == torch.float32 else dt)
            assert (out.cpu() - want).abs().max() < 3e-6
            if rows is not None:
                assert torch.equal(rows.cpu(), out.cpu().to(dt))


@pytest.mark.parametrize("width", [96, 100, 1000])
def test_norm_of_a_branch_added_into_the_stream(width):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(1)
    x = torch.randn(7, width, generator=g)
    y = torch.randn(7, width, generator=g) * 3
    w = 1 + 0.2 * torch.randn(width, generator=g)
    want = x.double() + plain.rms_norm(y.double(), 1e-5, w.double())
    resid = x.to(DEV).clone()
    rows = kernels.rmsnorm_add(resid, y.to(DEV), w.to(DEV), 1e-5, torch.bfloat16)
    assert (resid.cpu().double() - want).abs().max() < 2e-6 * want.abs().max()
    assert torch.equal(rows.cpu(), resid.cpu().to(torch.bfloat16))
    # a stack of partial sums, added in order; a bfloat16 branch; no norm at all
    parts = torch.randn(3, 7, width, generator=g)
    resid = x.to(DEV).clone()
    assert kernels.rmsnorm_add(resid, parts.to(DEV), w.to(DEV), 1e-5) is None
    want = x.double() + plain.rms_norm(parts.double().sum(0), 1e-5, w.double())
    assert (resid.cpu().double() - want).abs().max() < 2e-6 * want.abs().max()
    resid = x.to(DEV).clone()
    kernels.rmsnorm_add(resid, y.to(torch.bfloat16).to(DEV), w.to(DEV), 1e-5)
    want = x.double() + plain.rms_norm(y.to(torch.bfloat16).double(), 1e-5, w.double())
    assert (resid.cpu().double() - want).abs().max() < 2e-6 * want.abs().max()
    resid = x.to(DEV).clone()
    kernels.rmsnorm_add(resid, y.to(DEV), None, 0.0)
    assert torch.allclose(resid.cpu(), x + y)


def test_activations_times_up():
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(2)
    gu = torch.randn(9, 2 * 37, generator=g) * 3
    for act, f in (("gelu_tanh", plain.gelu_tanh), ("silu", plain.silu)):
        want = f(gu[:, :37].double()) * gu[:, 37:].double()
        got = kernels.act_mul(gu.to(DEV), act).cpu().double()
        assert (got - want).abs().max() < 1e-5
        got = kernels.act_mul(gu.to(torch.bfloat16).to(DEV), act).cpu().double()
        want = f(gu[:, :37].to(torch.bfloat16).double()) * gu[:, 37:].to(torch.bfloat16).double()
        assert (got - want).abs().max() < 0.02 * want.abs().max()


@pytest.mark.parametrize("M", [2, 8, 33])
def test_gate_up_product_with_the_activation_inside(M):
    """The tiled gate/up product of decode steps applies the tanh form of gelu as it applies silu."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(M)
    x = torch.randn(M, 192, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * 104, 192, generator=g) * 0.2).to(torch.bfloat16)
    for act, f in (("gelu_tanh", plain.gelu_tanh), ("silu", plain.silu)):
        want = f(x.double() @ w[:104].double().T) * (x.double() @ w[104:].double().T)
        got = kernels.linear_mid_gated(x.to(DEV), w.to(DEV), act=act).cpu().double()
        assert (got - want).abs().max() < 0.02 * want.abs().max()


def _pools(L, G, d, dv, page, dtype, grouped, seed=0):
    """Empty K and V pools with more pages than L tokens need, and a block table of shuffled pages."""
    n_pages = -(-L // page)
    order = list(range(n_pages + 3))
    random.Random(seed).shuffle(order)
    table = torch.tensor([order[:n_pages]], dtype=torch.int32)
    k_pool = torch.zeros(n_pages + 3, G, page, d, dtype=dtype)
    v_pool = torch.zeros((n_pages + 3, G, page // 8, dv, 8) if grouped else (n_pages + 3, G, page, dv), dtype=dtype)
    slots = torch.tensor([order[p // page] * page + p % page for p in range(L)], dtype=torch.int64)
    return k_pool, v_pool, table, slots


def _read_pools(k_pool, v_pool, table, L, grouped):
    page = k_pool.shape[2]
    k = torch.stack([k_pool[table[0, p // page], :, p % page] for p in range(L)])
    if grouped:
        v = torch.stack([v_pool[table[0, p // page], :, (p % page) // 8, :, p % 8] for p in range(L)])
    else:
        v = torch.stack([v_pool[table[0, p // page], :, p % page] for p in range(L)])
    return k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv", [(6, 2, 16, 24), (3, 3, 32, 8), (4, 1, 48, 48)])
def test_projection_rows_norm_blend_and_cache_write(H, G, d, dv, dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    grouped = dt == torch.bfloat16
    g = torch.Generator().manual_seed(3)
    L, page = 37, 8
    qkv = (torch.randn(L, H * d + G * d + G * dv, generator=g) * 2).to(dt)
    other = torch.randn(L, 5 + G * dv, generator=g).to(dt)           # the other values: a strided view of wider rows
    qw, kw = 1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped)
    slots[5] = -1                                                         # stores nothing
    other_dev = other.to(DEV)
    q = kernels.qkv_rows(qkv.to(DEV), qw.to(DEV), kw.to(DEV), 1e-5, slots.to(DEV), k_pool_d := k_pool.to(DEV),
                         v_pool_d := v_pool.to(DEV), H, G, d, dv, v_grouped=grouped, v_other=other_dev[:, 5:], mix=0.3)
    x = qkv.double()
    want_q = plain.rms_norm(x[:, :H * d], 1e-5, qw.double())
    want_k = plain.rms_norm(x[:, H * d:H * d + G * d], 1e-5, kw.double())
    want_v = plain.blend_values(x[:, H * d + G * d:], other[:, 5:].double(), 0.3)
    tol = 1e-5 if dt == torch.float32 else 1e-2
    assert (q.cpu().double().reshape(L, -1) - want_q).abs().max() < tol * want_q.abs().max()
    k, v = _read_pools(k_pool_d.cpu(), v_pool_d.cpu(), table, L, grouped)
    keep = [p for p in range(L) if p != 5]
    assert (k.double().reshape(L, -1)[keep] - want_k[keep]).abs().max() < tol * want_k.abs().max()
    assert (v.double().reshape(L, -1)[keep] - want_v[keep]).abs().max() < tol * want_v.abs().max()
    assert float(k[5].abs().max()) == 0 and float(v[5].abs().max()) == 0
    # no norm, no blend
    q = kernels.qkv_rows(qkv.to(DEV), None, None, 0.0, slots.to(DEV), k_pool_d, v_pool_d, H, G, d, dv, v_grouped=grouped)
    assert torch.equal(q.cpu().reshape(L, -1), qkv[:, :H * d])


def _planted(L, H, G, d, dv, window, softcap, scale, dtype, seed):
    """q, k, v of one sequence in which chosen (query, key) pairs have a score that stands far out:
    keys just inside and just outside the window, at page borders, the first token, far back."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(L, H, d, generator=g) * 0.3
    k = torch.randn(L, G, d, generator=g) * 0.3
    v = torch.randn(L, G, dv, generator=g)
    big = (softcap or 30.0) * 1.2 / scale
    pairs = []
    w = window or L
    for i in list(range(L - 12, L)) + [w - 1, w, w + 1, 17, 31, 32]:
        if not (0 <= i < L):
            continue
        for j in (i - w + 1, i - w, i - 15, i - 16, i - 17, 0, i - L // 2):
            if 0 <= j <= i:
                pairs.append((i, j))
    rng = random.Random(seed)
    for n, (i, j) in enumerate(pairs):
        h = rng.randrange(H)
        u = torch.zeros(d)
        u[n % d] = 1.0
        q[i, h] = u * (big ** 0.5)
        k[j, h // (H // G)] = u * (big ** 0.5)
    return q.to(dtype), k.to(dtype), v.to(dtype)


ATTN_CASES = [  # H, G, d, dv, window, softcap, scale, L
    (4, 2, 16, 24, 12, 20.0, 0.3, 70),
    (6, 2, 32, 16, 21, None, 0.2, 90),
    (3, 3, 64, 64, None, 35.0, 0.125, 150),
    (8, 2, 64, 128, 44, 45.0, 0.11, 200),
    (4, 4, 128, 64, 100, 30.0, 0.09, 330),
    (5, 1, 48, 80, 64, 30.0, 0.15, 130),
]


def _attention_case(case, dtype, fn, page=16, decode_tail=9):
    """Runs `fn` (a kernel binding taking the common operands) on a planted sequence: most of it as one
    portion, its last tokens one by one; compares with the plain attention of the whole sequence."""
    from xinfer_amd import kernels  # noqa: F401
    H, G, d, dv, window, softcap, scale, L = case
    dt = TD[dtype]
    grouped = dt == torch.bfloat16
    q, k, v = _planted(L, H, G, d, dv, window, softcap, scale, dt, seed=L)
    want = plain.attend(q.double(), k.double(), v.double(), scale, softcap, window)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, page, dt, grouped, seed=L)
    for p in range(L):
        pg, off = int(slots[p]) // page, int(slots[p]) % page
        k_pool[pg, :, off] = k[p]
        if grouped:
            v_pool[pg, :, off // 8, :, off % 8] = v[p]
        else:
            v_pool[pg, :, off] = v[p]
    slopes = torch.tensor([plain.head_slope(h, H) for h in range(H)], dtype=torch.float32).to(DEV)
    k_pool, v_pool, table = k_pool.to(DEV), v_pool.to(DEV), table.to(DEV)
    head = L - decode_tail
    outs = [fn(q[:head].to(DEV), k_pool, v_pool, table, list(range(head)), scale, window or 0, grouped, softcap or 0.0, slopes)]
    for p in range(head, L):
        outs.append(fn(q[p:p + 1].to(DEV), k_pool, v_pool, table, [p], scale, window or 0, grouped, softcap or 0.0, slopes))
    got = torch.cat([o.cpu() for o in outs]).double()
    tol = 2e-5 if dt == torch.float32 else 2e-2
    err = (got - want).abs().max(dim=1).values
    bad = (err > tol * want.abs().max()).nonzero()
    assert bad.numel() == 0, f"first wrong position {int(bad[0])} of {L} (window {window}): {float(err[int(bad[0])]):.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_generic_kernel_with_planted_keys(case, dtype):
    from xinfer_amd import kernels

    def fn(q, k_pool, v_pool, table, positions, scale, window, grouped, softcap, slopes):
        pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
        return kernels.attention_generic(q, k_pool, v_pool, table, torch.zeros_like(pos), pos, scale, window,
                                         v_grouped=grouped, softcap=softcap, slopes=slopes)
    _attention_case(case, dtype, fn)


@pytest.mark.parametrize("small", [None, 0, 1])
@pytest.mark.parametrize("case", ATTN_CASES + [(8, 1, 256, 128, 70, 25.0, 0.0625, 210), (2, 2, 32, 256, None, 25.0, 0.2, 190)])
def test_attention_matrix_core_kernel_with_planted_keys(case, small):
    """The bfloat16 kernel for scores with options: the same planted sequences, as a portion and token by
    token, in both workgroup shapes; also beside the generic kernel on the same operands."""
    from xinfer_amd import kernels
    H, G, d, dv = case[:4]
    assert kernels.attention_biased_supported(H, G, d, dv, 16)

    def fn(q, k_pool, v_pool, table, positions, scale, window, grouped, softcap, slopes):
        n, ctx = len(positions), positions[-1] + 1
        cu_q = torch.tensor([0, n], dtype=torch.int32, device=DEV)
        ctx_lens = torch.tensor([ctx], dtype=torch.int32, device=DEV)
        rows, shape = kernels.prefill_tiles([n], [ctx], d, H, G, small=small,
                                            block_of=lambda s_: kernels.attention_biased_block(d, dv, H // G, s_))
        tiles = torch.tensor(rows, dtype=torch.int32, device=DEV).reshape(-1, 2)
        split, span = 0, 0
        if n == 1 and small != 0:            # single tokens: also in slices of 64 or 128 keys put together afterwards
            span = min(ctx, window + 63) if window else ctx
            split = 64 if small is None else 128
        out = kernels.attention_biased_bf16(q, k_pool, v_pool, table, tiles, cu_q, ctx_lens, scale, window,
                                            softcap=softcap, slopes=slopes, small=shape, split_keys=split, span=span)
        pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
        ref = kernels.attention_generic(q, k_pool, v_pool, table, torch.zeros_like(pos), pos, scale, window,
                                        v_grouped=True, softcap=softcap, slopes=slopes)
        assert (out.float() - ref.float()).abs().max() <= 0.03 * ref.float().abs().max()
        return out
    _attention_case(case, "bfloat16", fn)


def test_slices_of_a_decode_step():
    from xinfer_amd import kernels
    assert kernels.biased_split_keys(1024, 4096) == 0                 # enough workgroups already
    assert kernels.biased_split_keys(64, 2048 + 63) == 320            # 8 slices asked for, 64-key steps
    assert kernels.biased_split_keys(8, 100) == 0                     # too few keys to cut
    assert kernels.biased_split_keys(1, 100000) % 64 == 0


def test_sizes_the_matrix_core_kernel_does_not_take():
    from xinfer_amd import kernels
    assert not kernels.attention_biased_supported(4, 4, 16, 12, 16)       # a value size that is no multiple of 8
    assert not kernels.attention_biased_supported(4, 4, 264, 16, 16)
    assert not kernels.attention_biased_supported(4, 3, 16, 16, 16)
    assert not kernels.attention_biased_supported(4, 4, 16, 16, 12)


def test_attention_without_the_options_is_the_plain_softmax():
    """No cap and no slopes: the kernel's options are off, not zero-valued."""
    from xinfer_amd import kernels
    H, G, d, dv, L = 4, 2, 16, 16, 40
    g = torch.Generator().manual_seed(5)
    q, k, v = torch.randn(L, H, d, generator=g), torch.randn(L, G, d, generator=g), torch.randn(L, G, dv, generator=g)
    want = plain.attend(q.double(), k.double(), v.double(), 0.25, None, None, biased=False)
    k_pool, v_pool, table, slots = _pools(L, G, d, dv, 8, torch.float32, False)
    for p in range(L):
        k_pool[int(slots[p]) // 8, :, int(slots[p]) % 8] = k[p]
        v_pool[int(slots[p]) // 8, :, int(slots[p]) % 8] = v[p]
    pos = torch.arange(L, dtype=torch.int32, device=DEV)
    got = kernels.attention_generic(q.to(DEV), k_pool.to(DEV), v_pool.to(DEV), table.to(DEV), torch.zeros_like(pos), pos, 0.25)
    assert (got.cpu().double() - want).abs().max() < 1e-5


@pytest.mark.parametrize("E,top,H", [(5, 2, 96), (3, 1, 100), (12, 2, 320), (7, 7, 64), (64, 6, 512)])
def test_router(E, top, H):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(E)
    x = torch.randn(33, H, generator=g)
    W = {"r.router": torch.randn(E, H, generator=g) * 0.3, "r.router.b": torch.randn(E, generator=g)}
    idx, wt = plain.route(x.double(), {k: t.double() for k, t in W.items()}, "r.", top)
    gi, gw = kernels.moe_route(x.to(DEV), W["r.router"].to(DEV), W["r.router.b"].to(DEV), top)
    assert torch.equal(gi.cpu().long(), idx)
    assert (gw.cpu().double() - wt).abs().max() < 1e-5
    assert (gw.sum(dim=1).cpu() - 1).abs().max() < 1e-5
    # equal logits: the lower index wins
    gi, gw = kernels.moe_route(torch.zeros(2, H, device=DEV), W["r.router"].to(DEV), None, top)
    assert gi.cpu().tolist() == [list(range(top))] * 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,H,F,T", [(5, 2, 96, 48, 19), (3, 1, 100, 24, 5), (8, 2, 512, 128, 70), (4, 4, 64, 200, 1)])
def test_experts(E, top, H, F, T, dtype):
    from xinfer_amd import kernels
    dt = TD[dtype]
    g = torch.Generator().manual_seed(F)
    x = torch.randn(T, H, generator=g).to(dt)
    W = {"r.router": torch.randn(E, H, generator=g) * 0.3, "r.router.b": torch.randn(E, generator=g)}
    for e in range(E):
        W[f"r.e{e}.gate"] = (torch.randn(F, H, generator=g) * 0.1).to(dt)
        W[f"r.e{e}.up"] = (torch.randn(F, H, generator=g) * 0.1).to(dt)
        W[f"r.e{e}.down"] = (torch.randn(H, F, generator=g) * 0.1).to(dt)
    ml = {"router": {"experts": E, "top": top}}
    want = plain.experts_ff(x.double(), {k: t.double() for k, t in W.items()}, "r.", ml)
    gi, gw = kernels.moe_route(x.to(DEV), W["r.router"].to(DEV), W["r.router.b"].to(DEV), top)
    gu = torch.stack([torch.cat([W[f"r.e{e}.gate"], W[f"r.e{e}.up"]]) for e in range(E)]).to(DEV)
    dn = torch.stack([W[f"r.e{e}.down"] for e in range(E)]).to(DEV)
    got = kernels.moe_experts(x.to(DEV), gu, dn, gi, gw, "silu")
    assert got.dtype == torch.float32
    tol = 1e-5 if dt == torch.float32 else 2e-2
    assert (got.cpu().double() - want).abs().max() < tol * want.abs().max()


@pytest.mark.parametrize("E,top,H,F,T", [(5, 2, 96, 48, 19), (3, 1, 104, 24, 5), (8, 2, 512, 128, 70), (4, 4, 64, 200, 1),
                                         (12, 3, 320, 72, 700), (2, 1, 64, 64, 300), (64, 6, 128, 32, 33)])
def test_experts_grouped_on_the_matrix_cores(E, top, H, F, T):
    """The grouped form against the plain implementation and against a pair at a time: tiles that are full, ragged
    and empty (experts nobody chose), both tile heights."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(F + T)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    W = {"r.router": torch.randn(E, H, generator=g) * 0.3, "r.router.b": torch.randn(E, generator=g)}
    if E == 12:
        W["r.router.b"][3] = -100.0          # an expert without rows
    for e in range(E):
        W[f"r.e{e}.gate"] = (torch.randn(F, H, generator=g) * 0.1).to(torch.bfloat16)
        W[f"r.e{e}.up"] = (torch.randn(F, H, generator=g) * 0.1).to(torch.bfloat16)
        W[f"r.e{e}.down"] = (torch.randn(H, F, generator=g) * 0.1).to(torch.bfloat16)
    gi, gw = kernels.moe_route(x.to(DEV), W["r.router"].to(DEV), W["r.router.b"].to(DEV), top)
    gu = torch.stack([torch.cat([W[f"r.e{e}.gate"], W[f"r.e{e}.up"]]) for e in range(E)]).to(DEV)
    dn = torch.stack([W[f"r.e{e}.down"] for e in range(E)]).to(DEV)
    one = kernels.moe_experts(x.to(DEV), gu, dn, gi, gw, "silu", grouped=False)
    got = kernels.moe_experts(x.to(DEV), gu, dn, gi, gw, "silu", grouped=True)
    assert (got - one).abs().max() <= 0.02 * one.abs().max()
    lib_out = kernels.moe_experts_library(x.to(DEV), gu, dn, gi, gw, "silu")          # the vendor library's products an expert
    assert (lib_out - one).abs().max() <= 0.02 * one.abs().max()
    for rows in (32, 64, 128):                   # every tile height gives a row the same sums
        again = kernels.moe_experts(x.to(DEV), gu, dn, gi, gw, "silu", grouped=True, tile_rows=rows)
        assert torch.equal(again, got), f"tiles of {rows} rows"
    if T <= 100:
        want = plain.experts_ff(x.double(), {k: t.double() for k, t in W.items()}, "r.", {"router": {"experts": E, "top": top}})
        assert (got.cpu().double() - want).abs().max() < 2e-2 * want.abs().max()
    assert not kernels.moe_grouped_takes(T, top, E, H + 4, F, torch.bfloat16, force=True)
    assert not kernels.moe_grouped_takes(T, top, E, H, F, torch.float32, force=True)


# ---- whole models ---------------------------------------------------------------------------------
LENGTHS = {"P": [1, 2, 12, 13, 33, 77, 130], "Q": [3, 9, 10, 18, 64, 101], "S": [1, 2, 3, 50, 90], "O": [1, 7, 8, 40, 75],
           "R": [5, 101, 330, 64, 301]}


def _requests(name):
    rng = random.Random(500 + ord(name))
    vocab = MODELS[name]["config"]["vocab"]
    return {f"r{i}": harness.random_prompt(rng, n, vocab) for i, n in enumerate(LENGTHS[name])}


_plain_cache = {}
_model_cache = {}


def _plain_logits(name, model_dir):
    if name not in _plain_cache:
        pm = plain.PlainMufenex(model_dir, torch.float64)
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
    runner = ModelRunner(model, page_size=page, num_pages=need // page, max_requests=4, **kw)     # exactly enough pages
    assert len(runner.cache.groups) == len({(l["mixer"].get("mask") or {}).get("size") for l in MODELS[name]["config"]["layers"]})
    got = harness.replay(runner, steps)
    for g in range(len(runner.cache.groups)):
        assert runner.cache.free_pages(g) == need // page
    rel = harness.compare(got, _plain_logits(name, dirs(name)), harness.TOL[dtype], f"{name}/{dtype}/{what}")
    print(f"{name}/{dtype}/{what}: worst error {rel:.2e} of the largest logit")
    return got, runner


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_whole(name, dtype, dirs):
    got, _ = _run(name, dtype, dirs, harness.trace_whole(_requests(name)), "whole")
    assert len(got) == sum(LENGTHS[name])


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
def test_mixed_batches_with_pages_used_again(name, dtype, dirs):
    for seed in (1, 2):
        _run(name, dtype, dirs, harness.trace_mixed(_requests(name), seed, max_live=3), f"mixed {seed}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q"])
def test_unequal_requests_decoding_together(name, dtype, dirs):
    reqs = {k: v for k, v in _requests(name).items() if len(v) > 8}
    reqs = dict(list(reqs.items())[:4])
    _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode", use_graphs=False)
    got, runner = _run(name, dtype, dirs, harness.trace_batch_decode(reqs, tail=7), "batch decode, graphs", graph_after=1)
    assert runner.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_passes_every_window_and_frees_pages(dtype, dirs):
    """Three tokens of prompt, then 150 one by one: every window passes over decoded tokens, pages of the
    windowed groups go back and come again while the request runs."""
    name = "P"
    rng = random.Random(9)
    toks = harness.random_prompt(rng, 153, MODELS[name]["config"]["vocab"])
    from xinfer_amd.engine import ModelRunner
    pm = plain.PlainMufenex(dirs(name), torch.float64)
    ref = {"a": pm.logits(toks).float()}
    steps = harness.trace_tail_one_by_one({"a": toks}, tail=150)
    page = MODELS[name]["page_size"]
    runner = ModelRunner(_model(name, dtype, dirs(name)), page_size=page, num_pages=[3, 4, 10], max_requests=2)
    windows = [g.window for g in runner.cache.groups]
    assert sorted(windows) == [0, 12, 21]
    got = harness.replay(runner, steps)
    harness.compare(got, ref, harness.TOL[dtype], f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_through_the_engine(dtype, dirs):
    """The framework's own entry point and scheduler: five prompts, three at a time, prompts cut into
    portions of 16 tokens, greedy tokens against the plain implementation."""
    from xinfer_amd import Engine, EngineConfig, SamplingParams
    name = "P"
    rng = random.Random(3)
    vocab = MODELS[name]["config"]["vocab"]
    prompts = [harness.random_prompt(rng, n, vocab) for n in (5, 40, 17, 33, 2)]
    eng = Engine(EngineConfig(weight_path=dirs(name), page_size=16, num_pages=24, max_num_seqs=3, prefill_chunk_size=16,
                              max_model_len=128, seed=1), dtype)
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    pm = plain.PlainMufenex(dirs(name), torch.float64)
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
    # the engine plans its own pages (three cache groups) where none are given
    rc = cli.main(["--w", dirs("P"), "--prompt-ids", "1,2,3,4,5,6,7,8,9", "--max-tokens", "4", "--max-model-len", "256",
                   "--temperature", "0", "--ignore-eos", "--page-size", "16", "--max-num-seqs", "4", "--dtype", "bf16"])
    assert rc == 0 and "Decoded tokens: 4 in" in capsys.readouterr().out
    rc = cli.main(["--w", dirs("Q"), "--prompt-ids", "1,2,3|4,5,6,7", "--max-tokens", "5", "--max-model-len", "64",
                   "--temperature", "0", "--ignore-eos", "--page-size", "8", "--num-pages", "16", "--dtype", "f32"])
    out = capsys.readouterr().out
    assert rc == 0 and "Decoded tokens: 10 in" in out


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(dtype, dirs, tmp_path):
    name = "Q"
    vocab = MODELS[name]["config"]["vocab"]
    reqs = {f"r{i}": harness.random_prompt(random.Random(60 + i), n, vocab) for i, n in enumerate([33, 70, 5, 64, 100])}
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
    pm = plain.PlainMufenex(dirs(name), torch.float64)
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
    """float32: steps replayed from a recorded graph give the bits of the same steps launched one by one
    (the values blended in from another layer travel inside the step, also under a graph)."""
    from xinfer_amd.engine import ModelRunner, StepEntry
    name = "P"
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
