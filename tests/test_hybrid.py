"""The pre-norm stacks of state-space and windowed-attention mixers (Tibalorn) against the float64 restatement in oracle/hybrid.py:
every mechanism alone through the C ABI, then whole models through the engine's step function -- whole prompts, token-by-token
decoding, portions, mixed batches, reused pages and slots, crafted keys at every edge, greedy generation.  Small random
configurations of their own; `be` runs each test on the CPU twin and (gpu) on the MI355X."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import hybrid as OH
from tests.conftest import ROOT

F32, BF16, I32 = torch.float32, torch.bfloat16, torch.int32
TOL = {F32: 3e-5, BF16: 4e-2}


def dev(be, a, dtype=F32):
    return be.t(np.asarray(a, dtype=np.float32)).to(dtype).contiguous()


def ints(be, a):
    return be.t(np.asarray(a, dtype=np.int32))


def rel_err(got, want):
    """rms over the last axis of the difference (mean removed) relative to the rms of the reference"""
    d = np.asarray(got, dtype=np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d * d).mean(-1)) / (np.sqrt((w * w).mean(-1)) + 1e-30)).max())


def close(got, want, tol):
    return np.abs(np.asarray(got, dtype=np.float64) - want).max() <= tol * (1 + np.abs(want).max())


# ---- row-wise steps and epilogues ------------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("width", [6, 50, 300, 2048, 4100])
def test_add_layer_norm(be, dtype, width):
    rng = np.random.default_rng(width)
    rows, eps = 5, 1e-3
    x = rng.standard_normal((rows, width)).astype(np.float32) * 3 + 1
    y = rng.standard_normal((rows, width)).astype(np.float32)
    w, b = OH.bf16_round(1 + rng.standard_normal(width) * 0.2), OH.bf16_round(rng.standard_normal(width) * 0.2)
    x32, out = be.t(x), torch.zeros((rows, width), dtype=dtype, device=be.device)
    be.ext.add_layer_norm(x32, be.t(y), dev(be, w, dtype), dev(be, b, dtype), out, rows, eps)
    s = x.astype(np.float64) + y
    want = np.array([OH.layer_norm(s[r], w, b, eps) for r in range(rows)])
    assert close(be.n(x32), s, 1e-6)
    assert close(be.n(out.float()), want, 3e-6 if dtype is F32 else 1e-2)
    # no addition, gathered rows, no bias
    idx = np.array([4, 1, 4], dtype=np.int32)
    out2 = torch.zeros((3, width), dtype=F32, device=be.device)
    be.ext.add_layer_norm(x32, None, dev(be, w, dtype), None, out2, 3, eps, row_idx=be.t(idx))
    assert close(be.n(out2), np.array([OH.layer_norm(s[r], w, 0.0, eps) for r in idx]), 3e-6)
    # only the addition
    be.ext.add_layer_norm(x32, be.t(y), None, None, None, rows, eps)
    assert close(be.n(x32), s + y, 1e-6)


@pytest.mark.parametrize("dtype,M,N,K", [(F32, 1, 9, 40), (F32, 33, 66, 50), (BF16, 3, 7, 24), (BF16, 17, 40, 64), (BF16, 45, 300, 72),
                                         (BF16, 130, 150, 72), (BF16, 21, 19, 20)])
@pytest.mark.parametrize("epi", [0, 4, 5])
def test_dense_linear_bias_and_activations(be, dtype, M, N, K, epi):
    rng = np.random.default_rng(M * 1000 + N * 10 + K + epi)
    x, w = OH.bf16_round(rng.standard_normal((M, K))), OH.bf16_round(rng.standard_normal((N, K)) / math.sqrt(K) * 3)
    bias = rng.standard_normal(N).astype(np.float32)
    acc = x.astype(np.float64) @ w.astype(np.float64).T + bias
    cap = 1.5
    want = {0: acc, 4: np.maximum(acc, 0) ** 2, 5: OH.soft_cap(acc, cap)}[epi]
    y = torch.full((M, N), float("nan"), dtype=F32, device=be.device)
    be.ext.dense_linear(dev(be, x, dtype), dev(be, w, dtype), y, M, N, K, K, K, N, epi=epi, limit=cap, bias=be.t(bias))
    assert close(be.n(y), want, 2e-5)


# ---- state-space mixer -------------------------------------------------------------------------------------------------------------


def spans_of(be, lens):
    row0 = np.cumsum([0] + list(lens[:-1]))
    return ints(be, row0), ints(be, lens), len(lens), max(lens)


@pytest.mark.parametrize("taps", [1, 2, 4, 7, 12])
def test_causal_conv_over_spans_and_steps(be, taps):
    """two sequences in two slots fed in unequal portions (shorter and longer than the taps, one token, 40 tokens): every output
    equals the convolution over the sequence's whole history; a slot that is used again starts from zeros"""
    rng = np.random.default_rng(taps)
    C, ld, off = 70, 83, 9
    w, b = OH.bf16_round(rng.standard_normal((C, taps))), OH.bf16_round(rng.standard_normal(C))
    tail = torch.full((3, max(taps - 1, 1), C), 7.0, dtype=F32, device=be.device)          # stale values of an earlier user
    hist = {1: np.zeros((0, C)), 2: np.zeros((0, C))}
    for step in ([(1, 2), (2, 1)], [(2, 40), (1, 1)], [(1, 1)], [(1, 5), (2, 3)], [(2, 1)], [(1, 70), (2, 2)], [(2, 3)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        f = rng.standard_normal((rows, ld)).astype(np.float32)
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(len(hist[s]), len(hist[s]) + n) for s, n in step])
        out = torch.zeros((rows, C), dtype=F32, device=be.device)
        be.ext.conv_silu_rows(be.t(f), ld, off, dev(be, w), dev(be, b), out, tail, spans_of(be, lens), ints(be, seq), ints(be, pos), C, taps)
        got, r = be.n(out), 0
        for s, n in step:
            for _ in range(n):
                hist[s] = np.concatenate([hist[s], f[r:r + 1, off:off + C].astype(np.float64)])
                padded = np.concatenate([np.zeros((taps, C)), hist[s]])[-taps:]
                assert close(got[r], OH.causal_conv(list(padded), w.astype(np.float64), b.astype(np.float64)), 3e-6), (step, r)
                r += 1


@pytest.mark.parametrize("heads,groups,N,P", [(4, 2, 8, 8), (3, 1, 5, 48), (2, 2, 33, 6), (1, 1, 16, 64), (6, 3, 128, 64), (2, 1, 7, 100), (1, 1, 256, 128)])
def test_selective_scan_over_spans_and_steps(be, heads, groups, N, P):
    """portions of 1 .. 37 tokens of two sequences: the state carried in the slot gives what one pass over the whole sequence gives"""
    rng = np.random.default_rng(heads * 100 + N)
    ldc, ldf = heads * P + 2 * groups * N + 3, heads + 5
    dt_bias, a_log, D = (rng.standard_normal(heads).astype(np.float32) for _ in range(3))
    state = torch.full((3, heads, N, P), 5.0, dtype=F32, device=be.device)
    S = {0: np.zeros((heads, N, P)), 2: np.zeros((heads, N, P))}
    at = {0: 0, 2: 0}
    for step in ([(2, 3), (0, 1)], [(0, 37), (2, 1)], [(2, 1)], [(2, 17), (0, 2)]):
        lens = [n for _s, n in step]
        rows = sum(lens)
        c, f = rng.standard_normal((rows, ldc)).astype(np.float32), rng.standard_normal((rows, ldf)).astype(np.float32) * 2
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(at[s], at[s] + n) for s, n in step])
        y = torch.zeros((rows, heads * P), dtype=F32, device=be.device)
        be.ext.ssm_scan(be.t(c), ldc, 0, heads * P, heads * P + groups * N, be.t(f), ldf, 2, be.t(dt_bias), be.t(a_log), be.t(D), y, state,
                        spans_of(be, lens), ints(be, seq), ints(be, pos), heads, groups, N, P)
        got, r = be.n(y), 0
        for s, n in step:
            for _ in range(n):
                u = c[r, :heads * P].astype(np.float64).reshape(heads, P)
                B = c[r, heads * P:heads * P + groups * N].astype(np.float64).reshape(groups, N)
                Cm = c[r, heads * P + groups * N:heads * P + 2 * groups * N].astype(np.float64).reshape(groups, N)
                d = OH.softplus(f[r, 2:2 + heads].astype(np.float64) + dt_bias)
                for h in range(heads):
                    g = h // (heads // groups)
                    S[s][h] = math.exp(-math.exp(a_log[h]) * d[h]) * S[s][h] + d[h] * np.outer(B[g], u[h])
                    assert close(got[r, h * P:(h + 1) * P], S[s][h].T @ Cm[g] + D[h] * u[h], 2e-5), (step, r, h)
                r += 1
            at[s] += n
    assert close(be.n(state)[2], S[2], 2e-5) and (be.n(state)[1] == 5.0).all()


@pytest.mark.parametrize("heads,groups,N,P", [(4, 2, 8, 8), (2, 1, 128, 64), (3, 3, 12, 100), (1, 1, 32, 48), (1, 1, 256, 128)])
def test_chunked_scan_equals_the_recurrence(be, heads, groups, N, P):
    """portions of 1 .. 200 tokens (several chunks, chunks that end early) through the chunked form, mixed with the token-by-token form
    on the same slots: outputs and carried state equal the plain recurrence"""
    assert be.ext.ssm_scan_chunked_supported(N, P) and not be.ext.ssm_scan_chunked_supported(N + 1, P)
    rng = np.random.default_rng(heads * 100 + N)
    ldc, ldf = heads * P + 2 * groups * N, heads + 5
    dt_bias, a_log, D = (rng.standard_normal(heads).astype(np.float32) for _ in range(3))
    state = torch.full((3, heads, N, P), 5.0, dtype=F32, device=be.device)
    S = {0: np.zeros((heads, N, P)), 2: np.zeros((heads, N, P))}
    at = {0: 0, 2: 0}
    for chunked, step in ((True, [(2, 3), (0, 130)]), (False, [(0, 1), (2, 1)]), (True, [(2, 200), (0, 64)]), (True, [(0, 65)]), (False, [(2, 2)])):
        lens = [n for _s, n in step]
        rows = sum(lens)
        c, f = rng.standard_normal((rows, ldc)).astype(np.float32), rng.standard_normal((rows, ldf)).astype(np.float32) * 2
        seq = np.concatenate([[s] * n for s, n in step])
        pos = np.concatenate([np.arange(at[s], at[s] + n) for s, n in step])
        y = torch.zeros((rows, heads * P), dtype=F32, device=be.device)
        args = (be.t(c), ldc, 0, heads * P, heads * P + groups * N, be.t(f), ldf, 2, be.t(dt_bias), be.t(a_log), be.t(D), y, state, spans_of(be, lens))
        if chunked:
            chunk0 = np.cumsum([0] + [-(-n // 64) for n in lens])
            total = int(chunk0[-1])
            zbuf = torch.zeros((total, heads, N, P), dtype=F32, device=be.device)
            dbuf = torch.zeros((total, heads), dtype=F32, device=be.device)
            be.ext.ssm_scan_chunked(*args, (ints(be, chunk0[:-1]), 64, total), ints(be, seq), ints(be, pos), zbuf, dbuf, heads, groups, N, P)
        else:
            be.ext.ssm_scan(*args, ints(be, seq), ints(be, pos), heads, groups, N, P)
        got, r = be.n(y), 0
        for s, n in step:
            for _ in range(n):
                u = c[r, :heads * P].astype(np.float64).reshape(heads, P)
                B = c[r, heads * P:heads * P + groups * N].astype(np.float64).reshape(groups, N)
                Cm = c[r, heads * P + groups * N:].astype(np.float64).reshape(groups, N)
                d = OH.softplus(f[r, 2:2 + heads].astype(np.float64) + dt_bias)
                for h in range(heads):
                    g = h // (heads // groups)
                    S[s][h] = math.exp(-math.exp(a_log[h]) * d[h]) * S[s][h] + d[h] * np.outer(B[g], u[h])
                    assert close(got[r, h * P:(h + 1) * P], S[s][h].T @ Cm[g] + D[h] * u[h], 3e-5), (step, r, h)
                r += 1
            at[s] += n
    assert close(be.n(state)[2], S[2], 3e-5) and close(be.n(state)[0], S[0], 3e-5) and (be.n(state)[1] == 5.0).all()


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("dim,groups", [(24, 1), (24, 3), (600, 2), (4100, 1)])
def test_gated_group_norm(be, dtype, dim, groups):
    rng = np.random.default_rng(dim + groups)
    rows, ldz, eps = 4, dim + 7, 1e-4
    y, z = rng.standard_normal((rows, dim)).astype(np.float32), rng.standard_normal((rows, ldz)).astype(np.float32)
    w = OH.bf16_round(1 + rng.standard_normal(dim) * 0.3)
    out = torch.zeros((rows, dim), dtype=dtype, device=be.device)
    be.ext.gated_group_norm(be.t(y), be.t(z), ldz, dev(be, w, dtype), out, rows, dim, groups, eps)
    v = (y.astype(np.float64) * OH.silu(z[:, :dim].astype(np.float64))).reshape(rows, groups, -1)
    want = (v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)).reshape(rows, dim) * w
    assert close(be.n(out.float()), want, 3e-6 if dtype is F32 else 1e-2)


# ---- windowed attention: the kernels alone -------------------------------------------------------------------------------------------


def test_rotary_tables_blend_and_amplitude():
    from exllamav2_amd.window_attn import rotary_tables
    for rot in ({"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                {"base": 500000.0, "dims": 6, "scaling": {"factor": 2.5, "original": 4096, "fast": 32.0, "slow": 1.0}},
                {"base": 100.0, "dims": 8, "scaling": None}):
        f, amp = rotary_tables(rot["base"], rot["dims"], rot["scaling"], "cpu")
        wf, wamp = OH.rotary_frequencies(rot)
        assert np.abs(f.numpy() - wf).max() <= 1e-7 * wf.max() and abs(amp - wamp) < 1e-12
    # the blend really differs from both pure forms somewhere
    rot = {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    wf, _ = OH.rotary_frequencies(rot)
    plain, _ = OH.rotary_frequencies(dict(rot, scaling=None))
    assert (wf == plain).any() and np.isclose(wf, plain / 8).any() and ((wf < plain * 0.999) & (wf > plain / 8 * 1.001)).any()


class KernelAttention:
    """drives exl2_kv_rot_append + exl2_window_attn directly over a hand-made pool: positions are appended in steps, each row's
    output is returned as [heads, vdim]"""

    def __init__(self, be, dtype, m, page, pages, table):
        self.be, self.m, self.dtype, self.page = be, m, dtype, page
        H, G, dim, vd, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["pool"]
        z = lambda *s: torch.zeros(s, dtype=dtype, device=be.device)
        self.k, self.v = z(pages, page, G, dim), z(pages, page, G, vd)
        self.kp, self.vp = z(pages, -(-page // P), G, dim), z(pages, -(-page // P), G, vd)
        self.table = ints(be, table)
        from exllamav2_amd.window_attn import rotary_tables
        self.freq, self.amp = rotary_tables(m["rot"]["base"], m["rot"]["dims"], m["rot"]["scaling"], be.device)
        self.vfreq, _ = rotary_tables(m["rot"]["base"], vd, None, be.device)

    def step(self, q, k, v, gate, seq, pos, q_scale, sink, tiles=False):
        """q [rows, H, dim], k [rows, G, dim], v [rows, G, vd], gate [rows, H, vd] before rotation; tiles: the matrix-core kernel over
        tiles of <= 64 rows (the rows of a step are consecutive positions of one sequence here)"""
        be, m = self.be, self.m
        H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        rows = len(seq)
        f = np.concatenate([q.reshape(rows, -1), k.reshape(rows, -1), v.reshape(rows, -1), gate.reshape(rows, -1)], 1).astype(np.float32)
        ld = f.shape[1]
        fd, qo = be.t(f), torch.zeros((rows, H * dim), dtype=self.dtype, device=be.device)
        sq, ps = ints(be, seq), ints(be, pos)
        be.ext.kv_rot_append(fd, ld, 0, H * dim, (H + G) * dim, qo, be.t(q_scale), self.k, self.v, self.kp, self.vp, self.freq, self.amp,
                             m["rot"]["dims"], self.vfreq, True, False, sq, ps, self.table, self.page, m["mask"]["pool"], rows, H, G, dim, vd)
        out = torch.zeros((rows, H * vd), dtype=self.dtype, device=be.device)
        common = (qo, self.k, self.v, self.kp, self.vp, be.t(sink), fd, ld, (H + G) * dim + G * vd, self.vfreq, True, False, sq, ps, self.table,
                  self.page, m["mask"]["pool"], out)
        if tiles:
            assert be.ext.window_attn_tiles_supported(self.dtype, dim, vd)
            if rows == 1:                                         # a decoded token: the kernel that shares the keys among a group's heads
                nsplit = [1, 3, 2][pos[0] % 3]                    # (also with the key list dealt to several workgroups, some of them idle)
                part_o = torch.zeros((1, H, nsplit, vd), dtype=F32, device=be.device)
                part_ml = torch.zeros((1, H, nsplit, 2), dtype=F32, device=be.device)
                be.ext.window_attn_tiles(*common, (ints(be, [0]), None, 1), 1, H, G, dim, vd, m["mask"]["size"], nsplit=nsplit,
                                         part_o=part_o, part_ml=part_ml)
            else:
                size = 64
                row0 = list(range(0, rows, size))
                be.ext.window_attn_tiles(*common, (ints(be, row0), ints(be, [min(size, rows - r) for r in row0]), len(row0)), size, H, G, dim, vd,
                                         m["mask"]["size"])
        else:
            be.ext.window_attn(*common, rows, H, G, dim, vd, m["mask"]["size"])
        return be.n(out.float()).reshape(rows, H, vd)


def attention_rows_oracle(m, q, k, v, gate, q_scale, sink):
    """float64, position by position, from the oracle's own pieces: q [T, H, dim] ... -> [T, H, vdim]"""
    T = q.shape[0]
    H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    W = {"l0.mix.q": np.eye(H * dim), "l0.mix.q.b": np.zeros(H * dim), "l0.mix.temp": q_scale / m["scale"], "l0.mix.sink": sink,
         "l0.mix.g": np.zeros((H * vd, H * dim)), "l0.mix.o": np.eye(H * vd)}
    f, amp = OH.rotary_frequencies(m["rot"])
    fv = OH.value_frequencies(m["rot"]["base"], vd)
    kv, out = [], []
    for p in range(T):
        kv.append((np.stack([OH.turn_halves(k[p, g].astype(np.float64), m["rot"]["dims"], p * f, amp) for g in range(G)]),
                   np.stack([OH.turn_halves(v[p, g].astype(np.float64), vd, p * fv) for g in range(G)])))
        o = OH.attention_token(W, "l0", m, q[p].reshape(-1).astype(np.float64), p, kv)          # gate weights are zero: sigmoid = 1/2
        out.append(o.reshape(H, vd) * 2.0 * OH.sigmoid(gate[p].astype(np.float64)))
    return np.stack(out)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("shape", [dict(heads=4, kv_heads=2, dim=16, vdim=8, size=6, pool=3, dims=8, page=4),
                                   dict(heads=3, kv_heads=3, dim=6, vdim=10, size=1, pool=1, dims=6, page=5),
                                   dict(heads=2, kv_heads=1, dim=32, vdim=32, size=9, pool=4, dims=32, page=8, scaling=None),
                                   dict(heads=6, kv_heads=2, dim=10, vdim=4, size=5, pool=7, dims=2, page=3)])
def test_attention_kernels_against_the_oracle(be, dtype, shape):
    """random q / k / v over 45 positions, appended in steps of unequal size through scattered pages: every position's output equals
    the float64 form -- window edges, blocks that become visible, sink, rotation of keys and values, gate"""
    shape = dict(shape)
    page = shape.pop("page")
    m = OH.attn_mixer(**shape)["mixer"]
    rng = np.random.default_rng(shape["dim"] * 7 + shape["size"])
    T, H, G, dim, vd = 45, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rnd = lambda *s: OH.bf16_round(rng.standard_normal(s)) if dtype is BF16 else rng.standard_normal(s).astype(np.float32)
    q, k, v, gate = rnd(T, H, dim), rnd(T, G, dim), rnd(T, G, vd), rnd(T, H, vd)
    q_scale = (m["scale"] * (1 + 0.3 * rng.standard_normal(H))).astype(np.float32)
    sink = rng.standard_normal(H).astype(np.float32) * 2
    want = attention_rows_oracle(m, q, k, v, gate, q_scale.astype(np.float64), sink.astype(np.float64))
    pages = -(-T // page) + 3
    table = np.zeros((2, pages), dtype=np.int32)
    table[1, :] = rng.permutation(pages)                      # slot 1, pages in no order
    ka = KernelAttention(be, dtype, m, page, pages, table)
    got, at = [], 0
    for n in [1, 1, 2, 7, 1, 16, 3, 1, 1, 12]:
        sl = slice(at, at + n)
        got.append(ka.step(q[sl], k[sl], v[sl], gate[sl], [1] * n, list(range(at, at + n)), q_scale, sink))
        at += n
    assert at == T
    assert close(np.concatenate(got), want, 2e-5 if dtype is F32 else 3e-2)


@pytest.mark.parametrize("shape", [dict(heads=4, kv_heads=2, dim=32, vdim=32, size=40, pool=8, dims=16, page=16),
                                   dict(heads=2, kv_heads=1, dim=64, vdim=64, size=70, pool=16, dims=64, page=64, scaling=None),
                                   dict(heads=3, kv_heads=3, dim=128, vdim=64, size=33, pool=5, dims=32, page=7),
                                   dict(heads=2, kv_heads=2, dim=96, vdim=96, size=200, pool=64, dims=32, page=256),
                                   dict(heads=2, kv_heads=1, dim=64, vdim=128, size=1, pool=1, dims=2, page=3),
                                   dict(heads=34, kv_heads=2, dim=32, vdim=32, size=20, pool=6, dims=8, page=32),
                                   dict(heads=2, kv_heads=1, dim=128, vdim=128, size=50, pool=8, dims=64, page=32),
                                   dict(heads=2, kv_heads=2, dim=192, vdim=128, size=90, pool=32, dims=96, page=128, scaling=None),
                                   dict(heads=1, kv_heads=1, dim=256, vdim=256, size=30, pool=4, dims=32, page=16)])
def test_matrix_core_attention_against_the_oracle(be, shape):
    """the bfloat16 tile kernel over 230 positions fed in steps of 1 .. 100 rows (tiles that start inside windows, blocks and pages,
    single decoded rows, a step of more than one tile): every position's output equals the float64 form"""
    shape = dict(shape)
    page = shape.pop("page")
    m = OH.attn_mixer(**shape)["mixer"]
    rng = np.random.default_rng(shape["dim"] + shape["size"])
    T, H, G, dim, vd = 370, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rnd = lambda *s: OH.bf16_round(rng.standard_normal(s))
    q, k, v, gate = rnd(T, H, dim), rnd(T, G, dim), rnd(T, G, vd), rnd(T, H, vd)
    q_scale = (m["scale"] * (1 + 0.3 * rng.standard_normal(H))).astype(np.float32)
    sink = rng.standard_normal(H).astype(np.float32) * 2
    want = attention_rows_oracle(m, q, k, v, gate, q_scale.astype(np.float64), sink.astype(np.float64))
    pages = -(-T // page) + 2
    table = np.zeros((2, pages), dtype=np.int32)
    table[1, :] = rng.permutation(pages)
    ka = KernelAttention(be, BF16, m, page, pages, table)
    got, at = [], 0
    for n in [1, 1, 30, 1, 100, 17, 1, 63, 1, 14, 1, 140]:
        sl = slice(at, at + n)
        got.append(ka.step(q[sl], k[sl], v[sl], gate[sl], [1] * n, list(range(at, at + n)), q_scale, sink, tiles=True))
        at += n
    assert at == T
    assert close(np.concatenate(got), want, 3e-2)


@pytest.mark.parametrize("decoded", [False, True])
def test_one_key_that_stands_out_at_every_edge(be, decoded):
    """among 700 keys one has a score far above the rest and a value of its own; the query sits so that this key is the last inside
    the window, the first outside (unseen), in the block that has just become visible, in the block that is not yet, 650 tokens back
    in a pooled block, and first / last of a page"""
    m = OH.attn_mixer(heads=2, kv_heads=1, dim=8, vdim=4, size=40, pool=8, dims=4, scaling=None)["mixer"]
    page, T = 16, 700
    rng = np.random.default_rng(5)
    sink, q_scale = np.zeros(2, dtype=np.float32), np.full(2, 1.0, dtype=np.float32)
    cases = []
    for target, query in [(659, 698), (658, 698), (647, 694), (648, 694), (40, 690), (639, 660), (640, 660), (0, 39), (0, 40), (0, 47), (0, 46)]:
        k = rng.standard_normal((T, 1, 8)).astype(np.float32) * 0.1
        v = rng.standard_normal((T, 1, 4)).astype(np.float32) * 0.1
        q = rng.standard_normal((T, 2, 8)).astype(np.float32) * 0.1
        k[target, 0, 4:] = 6.0                                # the unrotated part carries the match
        q[query, :, 4:] = 6.0
        v[target, 0] = [50.0, -50.0, 25.0, 10.0]
        want = attention_rows_oracle(m, q[:query + 1], k[:query + 1], v[:query + 1], np.zeros((query + 1, 2, 4)), q_scale.astype(np.float64),
                                     sink.astype(np.float64))[query]
        toks, blocks = OH.visible(query, 40, 8)
        seen = target in toks or target // 8 in blocks
        assert (np.abs(want).max() > 0.5) == seen, (target, query)           # the case shows what it is meant to show
        pages = -(-T // page)
        ka = KernelAttention(be, F32, m, page, pages, np.arange(pages, dtype=np.int32)[None, ::-1].copy())
        n0 = query if decoded else max(query - 20, 0)
        if n0:
            ka.step(q[:n0], k[:n0], v[:n0], np.zeros((n0, 2, 4)), [0] * n0, list(range(n0)), q_scale, sink)
        got = ka.step(q[n0:query + 1], k[n0:query + 1], v[n0:query + 1], np.zeros((query + 1 - n0, 2, 4)), [0] * (query + 1 - n0),
                      list(range(n0, query + 1)), q_scale, sink)[-1]
        assert close(got, want, 2e-5), (target, query)
        cases.append(seen)
    assert any(cases) and not all(cases)


# ---- whole models through the engine ---------------------------------------------------------------------------------------------

CONFIGS = {
    # both mixers, sizes that differ per layer, grouped state-space heads, a feed-forward behind a state-space layer
    "mixed": lambda: OH.small_config([
        OH.layer(OH.ssm_mixer(heads=4, vdim=8, state=8, groups=2, norm_groups=2, conv=3)),
        OH.layer(OH.attn_mixer(heads=4, kv_heads=2, dim=16, vdim=8, size=6, pool=3, dims=8), ff=40),
        OH.layer(OH.ssm_mixer(heads=2, vdim=12, state=5, groups=1, norm_groups=3, conv=4), ff=24),
        OH.layer(OH.attn_mixer(heads=2, kv_heads=2, dim=8, vdim=16, size=4, pool=5, dims=8, scaling=None))]),
    # attention first, a window of one token with blocks of one, two taps, one head
    "odd": lambda: OH.small_config([
        OH.layer(OH.attn_mixer(heads=3, kv_heads=1, dim=6, vdim=10, size=1, pool=1, dims=2), ff=20),
        OH.layer(OH.ssm_mixer(heads=1, vdim=20, state=3, groups=1, norm_groups=1, conv=2)),
        OH.layer(OH.attn_mixer(heads=2, kv_heads=1, dim=12, vdim=6, size=50, pool=2, dims=12, base=500.0), ff=16),
        OH.layer(OH.ssm_mixer(heads=3, vdim=6, state=9, groups=3, norm_groups=1, conv=1))], width=28, vocab=50, softcap=0.0, embed_scale=1.0),
    # head sizes the matrix-core attention takes in bfloat16, state-space sizes the chunked scan takes
    "wide": lambda: OH.small_config([
        OH.layer(OH.attn_mixer(heads=4, kv_heads=2, dim=32, vdim=32, size=9, pool=4, dims=16), ff=48),
        OH.layer(OH.ssm_mixer(heads=2, vdim=16, state=12, groups=2, norm_groups=1, conv=4)),
        OH.layer(OH.attn_mixer(heads=2, kv_heads=1, dim=64, vdim=64, size=5, pool=2, dims=64, scaling=None))], width=48, vocab=70),
}


def make_engine(be, cfg, W, dtype, max_tokens, page=4, max_seqs=4, graphs=None):
    from exllamav2_amd.config import LayeredConfig
    from exllamav2_amd.engine import Engine
    from exllamav2_amd.layered import LayeredModel
    tensors = {k: be.t(v).to(BF16) for k, v in W.items()}
    model = LayeredModel(LayeredConfig.from_dict_prenorm(cfg), device=be.device, dtype=dtype, ext=be.ext).load(tensors)
    return Engine(model, max_tokens=max_tokens, max_seqs=max_seqs, page_size=page, graphs=graphs)


def run_cuts(be, eng, rid, tokens, cuts):
    out, at = [], 0
    for c in cuts:
        out.append(be.n(eng.step([(rid, tokens[at:at + c], list(range(c)))])))
        at += c
    assert at == len(tokens)
    return np.concatenate(out, 0)


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_whole_prompt_and_residual_stream(be, name, dtype):
    cfg = CONFIGS[name]()
    W = OH.random_model(cfg, seed=1)
    toks = list(np.random.default_rng(2).integers(0, cfg["vocab"], size=23))
    want = OH.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, dtype, 32)
    assert rel_err(run_cuts(be, eng, "a", toks, [23]), want) <= TOL[dtype]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decoding_and_portions(be, name):
    """the same positions through a whole prompt, token by token from the first token on (windows, blocks and the recurrent state
    pass over decoded tokens), and in portions down to two tokens that end inside pages, windows, blocks and the taps"""
    cfg = CONFIGS[name]()
    W = OH.random_model(cfg, seed=3)
    toks = list(np.random.default_rng(4).integers(0, cfg["vocab"], size=26))
    want = OH.Oracle(cfg, W).feed("a", toks)
    for cuts in ([1] * 26, [2, 3, 2, 5, 2, 1, 1, 4, 2, 2, 2], [9] + [1] * 17, [25, 1], [1, 25]):
        eng = make_engine(be, cfg, W, F32, 28, page=4)
        assert rel_err(run_cuts(be, eng, "a", toks, cuts), want) <= TOL[F32], cuts


def test_mixed_batches_reuse_pages_and_slots(be):
    """five unequal requests over four slots and a pool smaller than their sum: portions beside single tokens, a request left out of
    a step, finished requests' pages and slot (with its recurrent state) taken by the next; every position equals the request alone"""
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=5)
    rng = np.random.default_rng(6)
    reqs = {r: list(rng.integers(0, cfg["vocab"], size=n)) for r, n in (("a", 13), ("b", 5), ("c", 9), ("d", 2), ("e", 11))}
    oracle = OH.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, F32, max_tokens=32, page=4, max_seqs=4)
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 3), ("c", 4), ("d", 2)], [("a", 2), ("c", 1)], [("c", 2), ("e", 3), ("a", 1)],
            [("a", 4), ("e", 2), ("c", 2)], [("e", 1)], [("e", 5)]]
    at, got = {r: 0 for r in reqs}, {r: [] for r in reqs}
    slots_used = {}
    for step in plan:
        entries, end = [], []
        for r, n in step:
            entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        for r, _n in step:
            if r in eng.slots:
                slots_used[r] = eng.slots[r]
        lg = be.n(eng.step(entries, end))
        for r, _n in step:
            slots_used.setdefault(r, eng.slots.get(r, slots_used.get(r)))
        k = 0
        for r, n in step:
            got[r].append(lg[k:k + n])
            k += n
    assert all(at[r] == len(reqs[r]) for r in reqs)
    assert len(eng.pool.free_pages) == eng.pool.num_pages and len(eng.pool.free_slots) == 4
    assert sum(-(-len(t) // 4) for t in reqs.values()) > eng.pool.num_pages            # pages were used again
    for r in reqs:
        assert rel_err(np.concatenate(got[r], 0), want[r]) <= TOL[F32], r


def test_a_reused_slot_starts_from_zeros(be):
    """one slot, three requests one after the other: the second and third find the first one's recurrent state, taps and pooled rows
    in their slot and pages and must not see them"""
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=15)
    rng = np.random.default_rng(16)
    eng = make_engine(be, cfg, W, F32, max_tokens=16, page=4, max_seqs=1)
    for r, n, cuts in (("a", 14, [14]), ("b", 9, [1, 1, 7]), ("c", 12, [2, 10])):
        toks = list(rng.integers(0, cfg["vocab"], size=n))
        want = OH.Oracle(cfg, W).feed(r, toks)
        assert rel_err(run_cuts(be, eng, r, toks, cuts), want) <= TOL[F32], r
        eng.finish(r)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_decode_steps_as_graphs(be, dtype):
    """decoding steps through the engine's persistent-input path (on a GPU: captured once per batch size and replayed; every replay
    is checked): two requests decode side by side, one ends, the other goes on alone, a third joins"""
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=21)
    rng = np.random.default_rng(22)
    reqs = {r: list(map(int, rng.integers(0, cfg["vocab"], size=n))) for r, n in (("a", 14), ("b", 9), ("c", 8))}
    oracle = OH.Oracle(cfg, W)
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
        assert rel_err(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r]) <= TOL[dtype], r
    eng.close()


def test_decode_graphs_survive_a_larger_step(be):
    """decode-only steps are captured while the scratch buffers are still small; a longer portion then moves the buffers; the decode
    steps after it must not replay the old addresses"""
    cfg = CONFIGS["wide"]()
    W = OH.random_model(cfg, seed=41)
    rng = np.random.default_rng(42)
    reqs = {r: list(map(int, rng.integers(0, cfg["vocab"], size=n))) for r, n in (("a", 12), ("b", 90), ("c", 10))}
    oracle = OH.Oracle(cfg, W)
    want = {r: oracle.feed(r, t) for r, t in reqs.items()}
    eng = make_engine(be, cfg, W, BF16, max_tokens=160, page=16, graphs=True)
    got = {r: {} for r in reqs}

    def step(parts, end=()):
        lg = be.n(eng.step([(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts], end))
        k = 0
        for r, lo, hi in parts:
            for p in range(lo, hi):
                got[r][p] = lg[k]; k += 1

    for i in range(5):
        step([("a", i, i + 1)])                                  # one token per step from the first token on: captured at the third
    step([("b", 0, 80), ("a", 5, 6)])                            # 81 rows: every scratch buffer grows
    for i in range(6, 12):
        step([("a", i, i + 1)])
    for i in range(80, 90):
        step([("b", i, i + 1), ("c", i - 80, i - 79)])
    for r in reqs:
        assert rel_err(np.stack([got[r][p] for p in range(len(reqs[r]))]), want[r]) <= TOL[BF16], r
    eng.close()


def crafted_model(window, pool, seed=31):
    """one attention layer between a state-space layer and a feed-forward, made so that token 0's query matches token 1's key and
    nothing else: queries read inputs 0-3, keys inputs 4-7 through the same matrix, values the other inputs; token 0 is marked in
    inputs 0-3, token 1 in 4-7, all other tokens are small there.  Wherever the mask lets token 0 see a token 1 -- as a token or
    inside a pooled block -- that key takes the softmax."""
    cfg = OH.small_config([OH.layer(OH.ssm_mixer(heads=2, vdim=8, state=4, groups=1, norm_groups=1, conv=2)),
                           OH.layer(OH.attn_mixer(heads=2, kv_heads=2, dim=8, vdim=8, size=window, pool=pool, dims=2, scaling=None, scale=0.75 * pool), ff=24)],
                          width=16, vocab=40, embed_scale=2.0)
    W = OH.random_model(cfg, seed=seed)
    rng = np.random.default_rng(seed + 1)
    E = W["embed"]
    E[:, :8] = 0.0
    mark = rng.standard_normal(4) * 2
    E[0, :4], E[1, 4:8] = mark, mark
    E[:, 8:] -= E.mean(1, keepdims=True) * 2                  # rows of mean zero: the layer norm leaves the unmarked inputs at zero
    W["embed"] = OH.bf16_round(E)
    M = rng.standard_normal((16, 4))
    W["l1.mix.q"], W["l1.mix.k"] = np.zeros((16, 16), dtype=np.float32), np.zeros((16, 16), dtype=np.float32)
    W["l1.mix.q"][:, :4], W["l1.mix.k"][:, 4:8] = OH.bf16_round(M), OH.bf16_round(M)
    W["l1.mix.q.b"][:], W["l1.mix.k.b"][:] = 0.0, 0.0
    W["l1.mix.v"][:, :8] = 0.0
    W["l1.mix.v"] = OH.bf16_round(W["l1.mix.v"] * 4)
    W["l1.mix.temp"][:] = 1.0
    W["l1.norm1"][:], W["l1.norm1.b"][:] = 1.0, 0.0
    W["l0.mix.o"] = OH.bf16_round(W["l0.mix.o"] * 0.05)          # the attention's input is nearly the token's own embedding
    W["l0.mix.o"][:8] = 0.0
    return cfg, W


@pytest.mark.parametrize("window,pool,page", [(24, 4, 8), (150, 16, 64)])
def test_a_repeated_token_at_every_edge_through_the_engine(be, window, pool, page):
    """whole prompt, portions that end right at the edges, and decoding: the marked token's first occurrence sits just inside / just
    outside the window, in the newest visible block / the one not yet visible, far back, and across a page border"""
    cfg, W = crafted_model(window, pool)
    rng = np.random.default_rng(window)
    T = window * 2 + 3 * pool + 9
    query = T - 1
    changed = 0
    for target in sorted({query - window + 1, query - window, (query - window + 1) // pool * pool - 1, (query - window + 1) // pool * pool,
                          1, page - 1, page, 0}):
        toks = [int(t) for t in rng.integers(2, cfg["vocab"], size=T)]
        toks[target], toks[query] = 1, 0                      # the marked pair, nowhere else
        base = list(toks)
        base[target] = 2
        oracle = OH.Oracle(cfg, W)
        want = oracle.feed("t", toks)
        other = OH.Oracle(cfg, W).feed("t", base)[-1]
        tk, bl = OH.visible(query, window, pool)
        if target in tk or target // pool in bl:
            changed += rel_err(want[-1:], other[None]) > 0.02          # where it can be seen it matters
        plans = [[T], [query - window + 1, window - 1, 1], [T - 3, 2, 1], [T - window - 2] + [1] * (window + 2),
                 [target + 1] + [2] * ((T - target - 1) // 2) + [1] * ((T - target - 1) % 2)]
        for cuts in (plans if window < 100 else plans[1:4]):
            eng = make_engine(be, cfg, W, F32, max_tokens=T + page, page=page)
            got = run_cuts(be, eng, "t", toks, cuts)
            assert rel_err(got[-4:], want[-4:]) <= TOL[F32], (target, cuts[:3])
    assert changed >= 5


def test_long_decoding_bf16(be):
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=7)
    toks = list(np.random.default_rng(8).integers(0, cfg["vocab"], size=60))
    want = OH.Oracle(cfg, W).feed("a", toks)
    eng = make_engine(be, cfg, W, BF16, 64, page=8)
    assert rel_err(run_cuts(be, eng, "a", toks, [3] + [1] * 57), want) <= TOL[BF16]


def test_greedy_generation_through_the_generator(be):
    from exllamav2_amd.engine import Generator
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=9)
    rng = np.random.default_rng(10)
    prompts = [list(map(int, rng.integers(0, cfg["vocab"], size=n))) for n in (7, 3, 5, 4, 6)]
    eng = make_engine(be, cfg, W, F32, max_tokens=64, page=4, max_seqs=3)
    out = Generator(eng, chunk=3).generate(prompts, 6)
    oracle = OH.Oracle(cfg, W)
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
    W = OH.random_model(cfg, seed=11)
    save_file({k: torch.from_numpy(v).to(BF16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert read_config(str(tmp_path))[0] == "Tibalorn"
    model = load_model(str(tmp_path), device=be.device, dtype=F32, ext=be.ext)
    toks = [1, 5, 9, 2, 2, 7]
    got = be.n(Engine(model, 16, page_size=4).step([("x", toks, list(range(6)))]))
    assert rel_err(got, OH.Oracle(cfg, W).feed("x", toks)) <= TOL[F32]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_command_replays_steps(tmp_path, dtype):
    """bin/trace_run in a process of its own: steps on standard input, logits files and `done` lines out"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from safetensors.torch import save_file
    cfg = CONFIGS["mixed"]()
    W = OH.random_model(cfg, seed=12)
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
    oracle = OH.Oracle(cfg, W)
    wa, wb = oracle.feed("a", a), oracle.feed("b", b)
    tol = TOL[F32] if dtype == "float32" else TOL[BF16]
    assert rel_err(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), wa[[0, 289]]) <= tol
    assert rel_err(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1), wb[[7]]) <= tol
    assert rel_err(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1), np.stack([wb[8], wa[299]])) <= tol
