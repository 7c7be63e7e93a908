"""The unquantized layer-stack models (latent attention with a sliding window, dense and scored-MoE feed-forwards, post-norm
residual steps) against the float64 restatement in oracle/layered.py: every mechanism alone through the C ABI, then whole models
through the engine's step function -- whole prompts, token-by-token decoding, portions, mixed batches, reused pages and slots,
greedy generation.  Small random configurations of their own; `be` runs each test on the CPU twin and (gpu) on the MI355X."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import layered as OL
from tests.conftest import ROOT

F32, BF16 = torch.float32, torch.bfloat16


def bf16_exact(a):
    u = np.asarray(a, dtype=np.float32).view(np.uint32)
    return (((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)


def dev(be, a, dtype):
    return be.t(np.asarray(a, dtype=np.float32)).to(dtype).contiguous()


def rel_err(got, want):
    """rms over the last axis of the difference (mean removed) relative to the rms of the reference"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d * d).mean(-1)) / (np.sqrt((w * w).mean(-1)) + 1e-30)).max())


TOL = {F32: 3e-5, BF16: 4e-2}

# ---- dense linears ---------------------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype,M,N,K", [(F32, 1, 9, 40), (F32, 5, 70, 36), (F32, 13, 8, 21), (F32, 33, 66, 50), (F32, 70, 10, 8),
                                         (BF16, 1, 12, 64), (BF16, 3, 7, 24), (BF16, 16, 33, 40), (BF16, 17, 40, 64), (BF16, 45, 300, 72),
                                         (BF16, 100, 20, 8), (BF16, 21, 19, 20), (BF16, 4, 6, 10), (BF16, 130, 150, 72), (BF16, 70, 130, 200),
                                         (BF16, 260, 24, 40)])
@pytest.mark.parametrize("epi", [0, 1, 2, 3])
def test_dense_linear(be, dtype, M, N, K, epi):
    rng = np.random.default_rng(M * 1000 + N * 10 + K + epi)
    x, w = bf16_exact(rng.standard_normal((M, K))), bf16_exact(rng.standard_normal((N, K)) / math.sqrt(K))
    aux = rng.standard_normal((M, N)).astype(np.float32) * 2
    acc = x.astype(np.float64) @ w.astype(np.float64).T
    a64, lim = aux.astype(np.float64), 0.8
    g = np.minimum(a64, lim)
    want = [acc, acc * OL.sigmoid(a64), a64 * OL.sigmoid(a64) * acc, g * OL.sigmoid(1.702 * g) * (np.clip(acc, -lim, lim) + 1)][epi]
    for out_dtype in ([F32] if dtype is F32 else [F32, BF16]):
        y = torch.full((M, N), float("nan"), dtype=out_dtype, device=be.device)
        be.ext.dense_linear(dev(be, x, dtype), dev(be, w, dtype), y, M, N, K, K, K, N, aux=be.t(aux) if epi else None, ldaux=N,
                            epi=epi, limit=lim)
        got = be.n(y.float())
        tol = 2e-5 if out_dtype is F32 else 1e-2
        assert np.abs(got - want).max() <= tol * (1 + np.abs(want).max()), (dtype, out_dtype)


@pytest.mark.parametrize("dtype,rows", [(F32, 3), (BF16, 2), (BF16, 30), (F32, 20)])
def test_dense_linear_batched_over_heads(be, dtype, rows):
    """per-head slabs with strided operands: the absorbed key projection's and the value projection's call shapes"""
    rng = np.random.default_rng(rows)
    H, dim, rot, R = 3, 8, 4, 16
    q = bf16_exact(rng.standard_normal((rows, H * (dim + rot))))
    w = bf16_exact(rng.standard_normal((H, R, dim)))
    y = torch.zeros((rows, H, R), dtype=F32, device=be.device)
    be.ext.dense_linear(dev(be, q, dtype), dev(be, w, dtype), y, rows, R, dim, H * (dim + rot), dim, H * R, batch=H, sxb=dim + rot,
                        swb=R * dim, syb=R)
    want = np.einsum("rhd,hnd->rhn", q.reshape(rows, H, dim + rot)[:, :, :dim].astype(np.float64), w.astype(np.float64))
    assert np.abs(be.n(y) - want).max() <= 2e-5 * (1 + np.abs(want).max())


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("rows,top", [(2, 2), (5, 1), (30, 3)])
def test_dense_linear_expert_rows_and_groups(be, dtype, rows, top):
    """rows that name their slab (decoding) and per-expert row lists (many rows) give what a per-pair loop gives"""
    rng = np.random.default_rng(rows * 7 + top)
    E, N, K = 4, 24, 16
    x, w = bf16_exact(rng.standard_normal((rows, K))), bf16_exact(rng.standard_normal((E, N, K)) / 4)
    ids = np.stack([rng.permutation(E + 2)[:top] for _ in range(rows)]).astype(np.int32)     # E, E + 1: experts without weights
    pairs = rows * top
    want = np.zeros((pairs, N))
    for p in range(pairs):
        e = ids.reshape(-1)[p]
        if e < E:
            want[p] = w[e].astype(np.float64) @ x[p // top].astype(np.float64)
    xd, wd = dev(be, x, dtype), dev(be, w, dtype)
    # the router hands out exactly these ids when their logits stand out, in this order
    logits = np.full((rows, E + 2), -40.0, dtype=np.float32)
    for r in range(rows):
        for k in range(top):
            logits[r, ids[r, k]] = 10.0 - k
    cnt, off, lst = (torch.zeros((E,), dtype=torch.int32, device=be.device), torch.zeros((E,), dtype=torch.int32, device=be.device),
                     torch.zeros((pairs,), dtype=torch.int32, device=be.device))
    wts = torch.zeros((rows, top), dtype=F32, device=be.device)
    idd = torch.zeros((rows, top), dtype=torch.int32, device=be.device)
    be.ext.moe_route_scored(be.t(logits), None, idd, wts, rows, E + 2, top, 1.0, E, groups=(cnt, off, lst))
    assert (be.n(idd) == ids).all()
    y = torch.zeros((pairs, N), dtype=F32, device=be.device)
    be.ext.dense_linear(xd, wd, y, pairs, N, K, K, K, N, swb=N * K, w_sel=idd.view(-1), n_sel=E, x_div=top)
    assert np.abs(be.n(y) - want).max() <= 2e-5 * (1 + np.abs(want).max())
    y2 = torch.zeros((pairs, N), dtype=F32, device=be.device)
    be.ext.dense_linear(xd, wd, y2, pairs, N, K, K, K, N, batch=E, swb=N * K, groups=(cnt, off, lst), x_div=top)
    assert np.abs(be.n(y2) - want).max() <= 2e-5 * (1 + np.abs(want).max())
    c, o, l = be.n(cnt), be.n(off), be.n(lst)
    for e in range(E):
        assert list(l[o[e]:o[e] + c[e]]) == [p for p in range(pairs) if ids.reshape(-1)[p] == e]


# ---- row-wise steps --------------------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width", [8, 50, 300])
def test_embed_norms(be, dtype, width):
    rng = np.random.default_rng(width)
    rows, vocab, eps, alpha = 5, 11, 1e-3, 1.7
    table = bf16_exact(rng.standard_normal((vocab, width)))
    ids = rng.integers(0, vocab, size=rows).astype(np.int32)
    x32 = torch.zeros((rows, width), dtype=F32, device=be.device)
    xh = x32 if dtype is F32 else torch.zeros((rows, width), dtype=dtype, device=be.device)
    be.ext.embed_scale(dev(be, table, dtype), be.t(ids), x32, xh, 3.0)
    want = table[ids].astype(np.float64) * 3.0
    assert np.abs(be.n(x32) - want).max() <= 1e-6 * np.abs(want).max()
    y = rng.standard_normal((rows, width)).astype(np.float32)
    w = bf16_exact(rng.standard_normal(width) * 0.2)
    be.ext.post_norm(x32, xh, be.t(y), dev(be, w, dtype), rows, alpha, eps)
    want = np.array([OL.post_norm(alpha * want[r] + y[r].astype(np.float64), w.astype(np.float64), eps) for r in range(rows)])
    assert np.abs(be.n(x32) - want).max() <= 3e-6 * (1 + np.abs(want).max())
    assert np.abs(be.n(xh.float()) - want).max() <= (3e-6 if dtype is F32 else 1e-2) * (1 + np.abs(want).max())
    # a slice of wider rows, plain weight, gathered rows
    src = rng.standard_normal((rows, width + 6)).astype(np.float32)
    idx = np.array([3, 0, 3], dtype=np.int32)
    out = torch.zeros((3, width), dtype=F32, device=be.device)
    be.ext.rms_rows(be.t(src), width + 6, dev(be, w, dtype), False, out, width, 3, width, eps, row_idx=be.t(idx), x_off=2)
    want = np.array([OL.rms(src[i, 2:2 + width].astype(np.float64), eps) * w for i in idx])
    assert np.abs(be.n(out) - want).max() <= 3e-6 * (1 + np.abs(want).max())


@pytest.mark.parametrize("experts,identity,top", [(4, 2, 2), (5, 0, 1), (3, 3, 4), (70, 5, 6)])
def test_router_and_expert_mixture(be, experts, identity, top):
    rng = np.random.default_rng(experts + top)
    rows, width, n = 6, 10, experts + identity
    logits = rng.standard_normal((rows, n)).astype(np.float32) * 2
    corr = (rng.standard_normal(n) * 0.3).astype(np.float32)
    ids = torch.zeros((rows, top), dtype=torch.int32, device=be.device)
    wts = torch.zeros((rows, top), dtype=F32, device=be.device)
    be.ext.moe_route_scored(be.t(logits), be.t(corr), ids, wts, rows, n, top, 1.25, experts)
    gi, gw = be.n(ids), be.n(wts)
    W = {"l0.mlp.correction": corr.astype(np.float64)}
    x = rng.standard_normal((rows, width)).astype(np.float32)
    ey = rng.standard_normal((rows * top, width)).astype(np.float32)
    y_want = np.zeros((rows, width))
    for r in range(rows):
        s = OL.softmax(logits[r].astype(np.float64))
        choice = s + corr
        want_ids = sorted(range(n), key=lambda e: (-choice[e], e))[:top]
        assert sorted(gi[r]) == sorted(want_ids)
        chosen = np.array([s[e] for e in gi[r]])
        assert np.abs(gw[r] - chosen / (chosen.sum() + 1e-20) * 1.25).max() <= 1e-6
        for k in range(top):
            y_want[r] += gw[r, k] * (x[r] if gi[r, k] >= experts else ey[r * top + k])
    # the mixture inside the residual step
    w = np.zeros(width, dtype=np.float32)
    x32 = be.t(x)
    be.ext.post_norm(x32, None, None, be.t(w), rows, 0.5, 1e-5, moe=(be.t(ey), ids, wts, experts))
    want = np.array([OL.post_norm(0.5 * x[r].astype(np.float64) + y_want[r], w.astype(np.float64), 1e-5) for r in range(rows)])
    assert np.abs(be.n(x32) - want).max() <= 1e-5


# ---- the latent cache and its attention ----------------------------------------------------------------------------------------------


def _attend_rows(be, dtype, R, rot, dims, H, window, page, n_tokens, dkv, q, q_abs, rows_at, base=100.0, scale=0.3, tiles=None):
    """append n_tokens rows of one sequence (pages handed out in a scrambled order), then attend from the positions rows_at"""
    n_pages = -(-n_tokens // page) + 2
    order = list(range(n_pages))[::-1]
    table = np.zeros((2, n_pages), dtype=np.int32)
    table[1, :] = order
    cache = torch.zeros((n_pages, page, R + rot), dtype=dtype, device=be.device)
    inv = be.t(np.array([base ** (-2.0 * i / max(dims, 1)) for i in range(max(1, dims // 2))], dtype=np.float32))
    seq = be.t(np.full(n_tokens, 1, dtype=np.int32))
    pos = be.t(np.arange(n_tokens, dtype=np.int32))
    nw = np.ones(R, dtype=np.float32)
    bt = be.t(table)
    be.ext.latent_append(be.t(dkv), R + rot, dev(be, nw, dtype), 1e-6, n_tokens, R, rot, dims, inv, seq, pos, bt, page, cache)
    n = len(rows_at)
    out = torch.zeros((n, H, R), dtype=dtype, device=be.device)
    args = (dev(be, q, dtype), H * rot, rot, 0, be.t(q_abs), cache, page, be.t(np.full(n, 1, dtype=np.int32)),
            be.t(np.array(rows_at, dtype=np.int32)), bt, out)
    if tiles is None:
        be.ext.latent_attn(*args, n, H, R, rot, dims, inv, scale, window)
    elif tiles[0] == 16:                                         # rows_at are consecutive positions: tiles of <= 16 of them
        row0 = list(range(0, n, 16))
        be.ext.latent_attn_tiles(*args, be.t(np.array(row0, dtype=np.int32)), be.t(np.array([min(16, n - r) for r in row0], dtype=np.int32)),
                                 len(row0), 16, H, R, rot, dims, inv, scale, window)
    else:                                                        # every row a decoded token, keys split over tiles[1] workgroups
        ns = tiles[1]
        po = torch.zeros((n, H, ns, R), dtype=F32, device=be.device) if ns > 1 else None
        pm = torch.zeros((n, H, ns, 2), dtype=F32, device=be.device) if ns > 1 else None
        be.ext.latent_attn_tiles(*args, be.t(np.arange(n, dtype=np.int32)), None, n, 1, H, R, rot, dims, inv, scale, window,
                                 nsplit=ns, part_o=po, part_ml=pm)
    return be.n(out.float())


def _attend_oracle(R, rot, dims, H, window, dkv, q, q_abs, rows_at, base=100.0, scale=0.3):
    kv = [(OL.rms(d[:R].astype(np.float64), 1e-6), OL.rotate(d[R:].astype(np.float64), j, base, dims)) for j, d in enumerate(dkv)]
    out = np.zeros((len(rows_at), H, R))
    for a, p in enumerate(rows_at):
        lo = max(0, p - window + 1)
        for h in range(H):
            qr = OL.rotate(q[a, h * rot:(h + 1) * rot].astype(np.float64), p, base, dims)
            s = np.array([(q_abs[a, h].astype(np.float64) @ kv[j][0] + qr @ kv[j][1]) * scale for j in range(lo, p + 1)])
            pr = OL.softmax(s)
            out[a, h] = sum(pr[j - lo] * kv[j][0] for j in range(lo, p + 1))
    return out


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("R,rot,dims,H,window,page", [(16, 4, 4, 2, 5, 4), (24, 8, 4, 1, 1, 8), (40, 6, 6, 3, 300, 16), (8, 2, 2, 2, 9, 3)])
def test_latent_attention_random(be, dtype, R, rot, dims, H, window, page):
    rng = np.random.default_rng(R + window)
    n = 21
    dkv = bf16_exact(rng.standard_normal((n, R + rot)))
    rows_at = [0, 1, window - 1 if window - 1 < n else 2, min(window, n - 1), n - 2, n - 1]
    q = bf16_exact(rng.standard_normal((len(rows_at), H * rot)))
    q_abs = rng.standard_normal((len(rows_at), H, R)).astype(np.float32)
    got = _attend_rows(be, dtype, R, rot, dims, H, window, page, n, dkv, q, q_abs, rows_at)
    want = _attend_oracle(R, rot, dims, H, window, dkv, q, q_abs, rows_at)
    assert np.abs(got - want).max() <= (2e-5 if dtype is F32 else 3e-2)


@pytest.mark.parametrize("R,rot,dims,H,window,page,n", [(32, 8, 8, 3, 5, 4, 40), (64, 16, 8, 5, 37, 8, 75), (160, 8, 8, 17, 1000, 16, 70),
                                                         (32, 40, 40, 70, 33, 7, 50), (288, 8, 4, 2, 20, 16, 45), (128, 32, 32, 2, 40, 16, 70),
                                                         (256, 64, 48, 5, 64, 32, 66)])
@pytest.mark.parametrize("tiles", [(16, 1), (1, 1), (1, 3), (1, 8)])
def test_latent_attention_on_the_matrix_cores(be, R, rot, dims, H, window, page, n, tiles):
    """the bfloat16 tile kernels (portions: 16 positions x a head per wave; decoded tokens: a position x 16 heads per wave, keys split
    over workgroups) against the plain restatement: head counts that do not fill a wave, windows that end inside a key step,
    more splits than key steps, rotation over part of the rotated block"""
    rng = np.random.default_rng(R + window + tiles[1])
    dkv = bf16_exact(rng.standard_normal((n, R + rot)))
    rows_at = list(range(n - 21, n)) if tiles[0] == 16 else [0, 1, min(window, n - 1), n - 1]
    q = bf16_exact(rng.standard_normal((len(rows_at), H * rot)))
    q_abs = bf16_exact(rng.standard_normal((len(rows_at), H, R)) * 0.5)
    got = _attend_rows(be, BF16, R, rot, dims, H, window, page, n, dkv, q, q_abs, rows_at, tiles=tiles)
    want = _attend_oracle(R, rot, dims, H, window, dkv, q, q_abs, rows_at)
    assert np.abs(got - want).max() <= 3e-2


@pytest.mark.parametrize("tiles", [None, (16, 1), (1, 1), (1, 4)])
@pytest.mark.parametrize("many_rows", [False, True])
@pytest.mark.parametrize("window,page,n,target_back", [(7, 4, 30, 6), (7, 4, 30, 7), (8, 8, 33, 7), (8, 8, 33, 8), (300, 16, 290, 289),
                                                        (300, 16, 290, 272), (5, 5, 6, 4), (5, 5, 6, 5)])
def test_window_edge_stands_out(be, tiles, many_rows, window, page, n, target_back):
    """One key gets a score far above all others: `target_back` tokens behind the query.  Inside the window (target_back <
    window) the output IS that key's latent; one token outside it must not be seen at all.  Queries at the last position alone
    (a decoded token) or among many rows (a prompt's portion); targets at page borders, just inside / outside, and far back."""
    R, rot, dims, H = (16, 4, 4, 2) if tiles is None else (32, 8, 8, 2)
    if tiles is not None and (tiles[0] == 16) != many_rows:
        pytest.skip("portions go to the 16-position tiles, single tokens to the one-position tiles")
    dtype = F32 if tiles is None else BF16
    rng = np.random.default_rng(n + target_back)
    dkv = bf16_exact(rng.standard_normal((n, R + rot)))
    dkv[:, R:] = 0                                               # scores come from the latent part alone
    p = n - 1
    tgt = p - target_back
    c_t = OL.rms(dkv[tgt, :R].astype(np.float64), 1e-6)
    rows_at = list(range(max(0, p - 9), n)) if many_rows else [p]
    q = np.zeros((len(rows_at), H * rot), dtype=np.float32)
    q_abs = (rng.standard_normal((len(rows_at), H, R)) * 0.05).astype(np.float32)
    boost = 60.0 if tiles is None else 8.0                       # (bfloat16 cache rows: a smaller boost keeps the OTHER scores' rounding small)
    q_abs[-1, :, :] += (boost * c_t).astype(np.float32)          # score of the target ~ boost |c|^2 * scale >> the rest
    if tiles is not None:
        q_abs = bf16_exact(q_abs)
    got = _attend_rows(be, dtype, R, rot, dims, H, window, page, n, dkv, q, q_abs, rows_at, tiles=tiles)
    want = _attend_oracle(R, rot, dims, H, window, dkv, q, q_abs, rows_at)
    assert np.abs(got - want).max() <= (5e-5 if tiles is None else 0.1)
    if target_back < window:
        assert np.abs(got[-1] - c_t[None, :]).max() <= (1e-3 if tiles is None else 3e-2)
    else:
        assert np.abs(got[-1] - c_t[None, :]).max() > 0.2


# ---- whole models through the engine ------------------------------------------------------------------------------------------------

CONFIGS = {
    # own keys / shared keys, dense and MoE, sizes that differ per layer
    "mixed": lambda: OL.small_config([
        OL.layer(OL.mixer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=24, window=6), OL.dense(48)),
        OL.layer(OL.mixer(heads=3, dim=8, rot_dim=8, vdim=24, kv_rank=32, q_rank=16, window=4, kv_from=0), OL.moe(4, 2, 2, 24)),
        OL.layer(OL.mixer(heads=1, dim=24, rot_dim=4, vdim=8, kv_rank=16, q_rank=8, window=9, base=500.0), OL.moe(3, 0, 1, 16, limit=0.7, scale=1.0))]),
    # sizes that are not multiples of 8, rotation over part of the rotated block, a layer without feed-forward, window 1
    "odd": lambda: OL.small_config([
        OL.layer(OL.mixer(heads=3, dim=6, rot_dim=6, vdim=10, kv_rank=20, q_rank=12, window=3, dims=4), None),
        OL.layer(OL.mixer(heads=2, dim=10, rot_dim=2, vdim=6, kv_rank=12, q_rank=20, window=1), OL.moe(2, 3, 3, 10)),
        OL.layer(OL.mixer(heads=2, dim=10, rot_dim=2, vdim=6, kv_rank=12, q_rank=20, window=50, kv_from=1), OL.dense(20))],
        width=36, vocab=50, alpha=1.0, embed_scale=1.0, eps=1e-3),
}


def make_engine(be, cfg, W, dtype, max_tokens, page=4, max_seqs=4, graphs=None):
    from exllamav2_amd.config import LayeredConfig
    from exllamav2_amd.engine import Engine
    from exllamav2_amd.layered import LayeredModel
    tensors = {k: be.t(v).to(BF16) for k, v in W.items()}
    model = LayeredModel(LayeredConfig.from_dict(cfg), device=be.device, dtype=dtype, ext=be.ext).load(tensors)
    return Engine(model, max_tokens=max_tokens, max_seqs=max_seqs, page_size=page, graphs=graphs)


def run_cuts(be, eng, rid, tokens, cuts):
    out, at = [], 0
    for c in cuts:
        lg = eng.step([(rid, tokens[at:at + c], list(range(c)))])
        out.append(be.n(lg))
        at += c
    assert at == len(tokens)
    return np.concatenate(out, 0)


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_whole_prompt(be, name, dtype):
    cfg = CONFIGS[name]()
    W = OL.random_model(cfg, seed=1)
    toks = list(np.random.default_rng(2).integers(0, cfg["vocab"], size=19))
    want = OL.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, dtype, 32)
    assert rel_err(run_cuts(be, eng, "a", toks, [19]), want) <= TOL[dtype]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decoding_and_portions(be, name):
    """the same positions through a whole prompt, token by token from the first token on (every window passes over decoded
    tokens), and in portions down to two tokens that end inside pages and windows"""
    cfg = CONFIGS[name]()
    W = OL.random_model(cfg, seed=3)
    toks = list(np.random.default_rng(4).integers(0, cfg["vocab"], size=22))
    want = OL.Oracle(cfg, W).feed("a", toks)
    for cuts in ([1] * 22, [2, 3, 2, 5, 2, 1, 1, 4, 2], [9] + [1] * 13, [21, 1]):
        eng = make_engine(be, cfg, W, F32, 24, page=4)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts), want) <= TOL[F32], cuts


def test_mixed_batches_reuse_pages_and_slots(be):
    """five unequal requests over four slots and a pool smaller than their sum: portions beside single tokens, a request left out of
    a step, finished requests' pages and slot taken by the next; every position equals the request run alone"""
    cfg = CONFIGS["mixed"]()
    W = OL.random_model(cfg, seed=5)
    rng = np.random.default_rng(6)
    reqs = {r: list(rng.integers(0, cfg["vocab"], size=n)) for r, n in (("a", 13), ("b", 5), ("c", 9), ("d", 2), ("e", 11))}
    oracle = OL.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, F32, max_tokens=32, page=4, max_seqs=4)
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 3), ("c", 4), ("d", 2)], [("a", 2), ("c", 1)], [("c", 2), ("e", 3), ("a", 1)],
            [("a", 4), ("e", 2), ("c", 2)], [("e", 1)], [("e", 5)]]
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    pages_seen = set()
    for step in plan:
        entries, end = [], []
        for r, n in step:
            entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        lg = be.n(eng.step(entries, end))
        k = 0
        for r, n in step:
            got[r].append(lg[k:k + n])
            k += n
        pages_seen.add(eng.pool.num_pages - len(eng.pool.free_pages))
    assert all(at[r] == len(reqs[r]) for r in reqs)
    assert len(eng.pool.free_pages) == eng.pool.num_pages and len(eng.pool.free_slots) == 4
    assert sum(-(-len(t) // 4) for t in reqs.values()) > eng.pool.num_pages            # pages were used again
    for r in reqs:
        assert rel_err(np.concatenate(got[r], 0), want[r]) <= TOL[F32], r


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_decode_steps_as_graphs(be, dtype):
    """decoding steps through the engine's persistent-input path (on a GPU: captured once per batch size and replayed; every replay
    is checked): two requests decode side by side, one ends, the other goes on alone, a third joins"""
    cfg = CONFIGS["mixed"]()
    W = OL.random_model(cfg, seed=21)
    rng = np.random.default_rng(22)
    reqs = {r: list(map(int, rng.integers(0, cfg["vocab"], size=n))) for r, n in (("a", 14), ("b", 9), ("c", 8))}
    oracle = OL.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, dtype, max_tokens=48, page=4, graphs=True)
    got = {r: {} for r in reqs}

    def step(parts, end=()):
        lg = be.n(eng.step([(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts], end))
        k = 0
        for r, lo, hi in parts:
            for p in range(lo, hi):
                got[r][p] = lg[k]; k += 1

    step([("a", 0, 3), ("b", 0, 2)])
    for i in range(6):
        step([("a", 3 + i, 4 + i), ("b", 2 + i, 3 + i)])
    step([("b", 8, 9)], end=["b"])
    for i in range(3):
        step([("a", 9 + i, 10 + i)])
    step([("c", 0, 4)])
    for i in range(2):
        step([("c", 4 + i, 5 + i), ("a", 12 + i, 13 + i)])
    step([("c", 6, 8)], end=["c", "a"])
    for r in reqs:
        assert sorted(got[r]) == list(range(len(reqs[r])))
        # (bfloat16 on a tiny random model: a router score near a tie may pick another expert; a wrong slot or position shows as ~1)
        assert rel_err(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r]) <= (TOL[F32] if dtype is F32 else 0.1), r
    eng.close()


def test_long_decoding_bf16(be):
    cfg = CONFIGS["mixed"]()
    W = OL.random_model(cfg, seed=7)
    toks = list(np.random.default_rng(8).integers(0, cfg["vocab"], size=40))
    want = OL.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, BF16, 40, page=8)
    assert rel_err(run_cuts(be, eng, "a", toks, [3] + [1] * 37), want) <= TOL[BF16]


def test_greedy_generation_through_the_generator(be):
    from exllamav2_amd.engine import Generator
    cfg = CONFIGS["mixed"]()
    W = OL.random_model(cfg, seed=9)
    rng = np.random.default_rng(10)
    prompts = [list(map(int, rng.integers(0, cfg["vocab"], size=n))) for n in (7, 3, 5, 4, 6)]
    eng = make_engine(be, cfg, W, F32, max_tokens=64, page=4, max_seqs=3)
    out = Generator(eng, chunk=3).generate(prompts, 6)
    oracle = OL.Oracle(cfg, W)
    checked = 0
    for i, p in enumerate(prompts):
        lg = oracle.feed(i, p)[-1]
        for t in out[i]:
            top2 = np.sort(lg)[-2:]
            if top2[1] - top2[0] < 1e-3:
                break                                             # a near tie: later tokens may differ legitimately
            assert t == int(np.argmax(lg))
            checked += 1
            lg = oracle.feed(i, [t])[-1]
        assert len(out[i]) == 6
    assert checked >= 20
    assert len(eng.pool.free_pages) == eng.pool.num_pages


def test_model_directory_registry(be, tmp_path):
    """config.json + model.safetensors -> architectures.load_model picks the class by the architecture name"""
    from safetensors.torch import save_file
    from exllamav2_amd.architectures import load_model, read_config
    from exllamav2_amd.engine import Engine
    cfg = CONFIGS["odd"]()
    W = OL.random_model(cfg, seed=11)
    save_file({k: torch.from_numpy(v).to(BF16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert read_config(str(tmp_path))[0] == "Benolix"
    model = load_model(str(tmp_path), device=be.device, dtype=F32, ext=be.ext)
    toks = [1, 5, 9, 2, 2, 7]
    got = be.n(Engine(model, 16, page_size=4).step([("x", toks, list(range(6)))]))
    assert rel_err(got, OL.Oracle(cfg, W).feed("x", toks)) <= TOL[F32]
    bad = dict(cfg, architecture="NoSuchDesign")
    (tmp_path / "config.json").write_text(json.dumps(bad))
    with pytest.raises(RuntimeError, match="NoSuchDesign"):
        read_config(str(tmp_path))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_command_replays_steps(tmp_path, dtype):
    """bin/trace_run in a process of its own: steps on standard input, logits files and `done` lines out"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from safetensors.torch import save_file
    cfg = CONFIGS["mixed"]()
    W = OL.random_model(cfg, seed=12)
    mdir = tmp_path / "model"
    mdir.mkdir()
    save_file({k: torch.from_numpy(v).to(BF16) for k, v in W.items()}, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(cfg))
    rng = np.random.default_rng(13)
    a, b = list(map(int, rng.integers(0, cfg["vocab"], size=300))), list(map(int, rng.integers(0, cfg["vocab"], size=9)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:290], "want": [0, 289]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[290:295], "want": []}, {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": [0]}, {"id": "a", "tokens": a[295:], "want": [4]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dtype, "--out", str(out), "--max-tokens", "512"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600, cwd=str(tmp_path))
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    oracle = OL.Oracle(cfg, W)
    wa, wb = oracle.feed("a", a), oracle.feed("b", b)
    tol = TOL[F32] if dtype == "float32" else TOL[BF16]
    g0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)
    assert rel_err(g0, wa[[0, 289]]) <= tol
    g1 = np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)
    assert rel_err(g1, wb[[7]]) <= tol
    g2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)
    assert rel_err(g2, np.stack([wb[8], wa[299]])) <= tol


def test_engine_serves_the_quantized_family_too(be):
    """the same Engine.step / Generator over a quantized Llama-style model: its paged forward behind the engine's interface gives
    what its own contiguous-cache forward gives, in portions and decoding, two requests side by side"""
    from exllamav2_amd import ExLlamaV2, ExLlamaV2Cache, ExLlamaV2Config
    from exllamav2_amd.engine import Engine, Generator
    from exllamav2_amd.synth import synth_checkpoint
    cfg = ExLlamaV2Config.tiny_test(num_hidden_layers=2, max_seq_len=512, max_input_len=16)
    model = ExLlamaV2(cfg, device=be.device, ext=be.ext).load(synth_checkpoint(cfg, be.device, seed=3))
    rng = np.random.default_rng(3)
    a, b = rng.integers(0, cfg.vocab_size, size=9), rng.integers(0, cfg.vocab_size, size=5)
    want = {}
    for name, ids in (("a", a), ("b", b)):
        cache = ExLlamaV2Cache(model, batch_size=1)
        want[name] = be.n(model.forward(torch.from_numpy(ids[None, :]), cache, last_id_only=False).float())[0]
    eng = Engine(model, max_tokens=512, max_seqs=2)
    got = {"a": [], "b": []}
    for step in ([("a", 0, 4)], [("a", 4, 7), ("b", 0, 4)], [("a", 7, 8), ("b", 4, 5)], [("a", 8, 9)]):
        lg = be.n(eng.step([(r, list(map(int, {"a": a, "b": b}[r][lo:hi])), list(range(hi - lo))) for r, lo, hi in step]))
        k = 0
        for r, lo, hi in step:
            got[r].append(lg[k:k + hi - lo]); k += hi - lo
    for r in ("a", "b"):
        g = np.concatenate(got[r], 0)
        assert np.abs(g - want[r]).max() <= 0.06 + np.abs(want[r]).max() * 2.0 ** -7, r
    eng.finish("a"); eng.finish("b")
    out = Generator(eng, chunk=4).generate([list(map(int, a[:6])), list(map(int, b))], 3)
    assert [len(o) for o in out] == [3, 3]
    model.unload()
