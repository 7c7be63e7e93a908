"""Plain float64 restatement of the Tibalorn layer stack (state-space and windowed-attention mixers behind pre-norm residual
steps) -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, token by token, written from the equations; nothing is shared with the product path (no pages, no
slots, no batching, no pooled-row tables: a sequence's memory is python lists and per-layer arrays).

Notation: W x with W stored [out, in]; h = a sublayer's input; p = a token's position (from 0).
    layer:   x <- x + mixer(LN1(x));  x <- x + ff(LN2(x)) (absent when the layer has no feed-forward)
             LN(v) = (v - mean v) / sqrt(var v + eps) * w + b
    state-space mixer (selective scan with scalar decay per head):
             [z | u | B | C | d] = W_in h;  (u, B, C) <- silu(causal conv over the last `taps` tokens + bias), per channel
             d <- softplus(d + d_bias);  head i (group g = i // (heads / groups)):
             S_i <- exp(-exp(A_i) d_i) S_i + d_i B_g u_i^T;   y_i = S_i^T C_g + D_i u_i
             out = W_o (groupwise_rms(y * silu(z)) * w_norm)
    windowed attention (grouped heads, biases on q / k / v):
             q, k: first `dims` values of a head in pairs (i, i + dims / 2) turned by p * f_i (frequencies blended between
             f_i and f_i / factor by a ramp over i, amplitudes times 0.1 ln(factor) + 1)
             v: all values in pairs (m, m + vdim / 2) turned by p * base^(-2m / vdim); a head's output is turned back by -p
             keys seen from p: tokens j with 0 <= p - j < size, and the mean key / mean value of every block of `pool` tokens
             [bP, bP + P) with bP + P - 1 <= p - size
             weights: exp(s_j) / (exp(sink) + sum exp(s)),  s_j = q . k_j * scale * temp
             out = W_o (heads * sigmoid(W_g h))
    ff:      W_down relu(W_up h)^2
    logits:  c tanh(E LN_final(x) / c), E the embedding table (inputs are E[token] * embedding scale)
"""
from __future__ import annotations

import math

import numpy as np


def layer_norm(v, w, b, eps):
    d = v - v.mean()
    return d / math.sqrt(float(np.mean(d * d)) + eps) * w + b


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def causal_conv(history, taps_w, bias):
    """history: the channel vectors of the last `taps` tokens, oldest first (zeros before the sequence's start)"""
    taps = taps_w.shape[1]
    acc = bias.copy()
    for k in range(taps):
        acc = acc + taps_w[:, k] * history[k]
    return silu(acc)


def ssm_token(W, key, m, h, mem, eps):
    """mem: {"hist": list of the last taps - 1 conv inputs, "S": [heads, state, vdim]} -- updated in place"""
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    f = W[key + ".mix.in"] @ h
    z, xbc, d = f[:inner], f[inner:2 * inner + 2 * G * N], f[2 * inner + 2 * G * N:]
    taps = m["conv"]
    hist = mem["hist"] + [xbc]
    c = causal_conv(hist[-taps:], W[key + ".mix.conv"], W[key + ".mix.conv.b"])
    mem["hist"] = hist[1:] if taps > 1 else []
    u, B, C = c[:inner].reshape(H, P), c[inner:inner + G * N].reshape(G, N), c[inner + G * N:].reshape(G, N)
    d = softplus(d + W[key + ".mix.dt_bias"])
    y = np.zeros((H, P))
    for i in range(H):
        g = i // (H // G)
        decay = math.exp(-math.exp(W[key + ".mix.A_log"][i]) * d[i])
        mem["S"][i] = decay * mem["S"][i] + d[i] * np.outer(B[g], u[i])
        y[i] = mem["S"][i].T @ C[g] + W[key + ".mix.D"][i] * u[i]
    y = y.reshape(-1) * silu(z)
    parts = y.reshape(m["norm_groups"], -1)
    parts = parts / np.sqrt((parts * parts).mean(-1, keepdims=True) + eps)
    return W[key + ".mix.o"] @ (parts.reshape(-1) * W[key + ".mix.norm"])


def rotary_frequencies(rot):
    """(frequencies [dims / 2], amplitude) of the q / k rotation, with the blended long-context scaling if the layer has one"""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    def turn_dim(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def turn_halves(vec, n, angles, amp=1.0):
    """pairs (i, i + n / 2) of the first n values turned by angles[i]; the rest unchanged"""
    out = vec.copy()
    half = n // 2
    for i in range(half):
        c, s = math.cos(angles[i]) * amp, math.sin(angles[i]) * amp
        out[i] = vec[i] * c - vec[i + half] * s
        out[i + half] = vec[i + half] * c + vec[i] * s
    return out


def value_frequencies(base, vdim):
    return np.array([base ** (-2.0 * m / vdim) for m in range(vdim // 2)])


def attention_kv(W, key, m, h, pos):
    """what a cache keeps for one token: (keys [kv_heads, dim] rotated, values [kv_heads, vdim] rotated)"""
    G, dim, vd, rot = m["kv_heads"], m["dim"], m["vdim"], m["rot"]
    f, amp = rotary_frequencies(rot)
    k = (W[key + ".mix.k"] @ h + W[key + ".mix.k.b"]).reshape(G, dim)
    v = (W[key + ".mix.v"] @ h + W[key + ".mix.v.b"]).reshape(G, vd)
    fv = value_frequencies(rot["base"], vd)
    return (np.stack([turn_halves(k[g], rot["dims"], pos * f, amp) for g in range(G)]),
            np.stack([turn_halves(v[g], vd, pos * fv) for g in range(G)]))


def visible(pos, size, pool):
    """(token positions, block numbers) that position `pos` attends to"""
    tokens = list(range(max(0, pos - size + 1), pos + 1))
    blocks = [b for b in range(0, pos // pool + 1) if b * pool + pool - 1 <= pos - size]
    return tokens, blocks


def attention_token(W, key, m, h, pos, kv):
    """kv: list over positions 0..pos of attention_kv results (this token's included)"""
    H, G, dim, vd, rot = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["rot"]
    size, P = m["mask"]["size"], m["mask"]["pool"]
    f, amp = rotary_frequencies(rot)
    fv = value_frequencies(rot["base"], vd)
    q = (W[key + ".mix.q"] @ h + W[key + ".mix.q.b"]).reshape(H, dim)
    tokens, blocks = visible(pos, size, P)
    outs = []
    for i in range(H):
        g = i // (H // G)
        qi = turn_halves(q[i], rot["dims"], pos * f, amp)
        keys = [np.mean([kv[j][0][g] for j in range(b * P, b * P + P)], axis=0) for b in blocks] + [kv[j][0][g] for j in tokens]
        vals = [np.mean([kv[j][1][g] for j in range(b * P, b * P + P)], axis=0) for b in blocks] + [kv[j][1][g] for j in tokens]
        s = np.array([qi @ kk for kk in keys]) * m["scale"] * W[key + ".mix.temp"][i]
        sink = W[key + ".mix.sink"][i]
        top = max(s.max(), sink)
        e = np.exp(s - top)
        wts = e / (e.sum() + math.exp(sink - top))
        o = sum(w * v for w, v in zip(wts, vals))
        outs.append(turn_halves(o, vd, -pos * fv))
    o = np.concatenate(outs) * sigmoid(W[key + ".mix.g"] @ h)
    return W[key + ".mix.o"] @ o


def relu2_ff(W, key, h):
    a = np.maximum(W[key + ".mlp.up"] @ h, 0.0)
    return W[key + ".mlp.down"] @ (a * a)


def soft_cap(z, c):
    return c * np.tanh(z / c) if c else z


class Oracle:
    """feed(seq, tokens) -> logits [len(tokens), vocab] of the sequence's next tokens; state is kept per sequence name"""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.W = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.seqs = {}

    def _new(self):
        mem = []
        for spec in self.cfg["layers"]:
            m = spec["mixer"]
            if spec["type"] == "mamba2":
                ch = m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"]
                mem.append({"hist": [np.zeros(ch) for _ in range(m["conv"] - 1)], "S": np.zeros((m["heads"], m["state"], m["vdim"]))})
            else:
                mem.append([])
        return {"n": 0, "mem": mem}

    def feed(self, seq, tokens, residuals=None):
        cfg, W, eps = self.cfg, self.W, self.cfg["norm"]["eps"]
        st = self.seqs.setdefault(seq, None) or self._new()
        self.seqs[seq] = st
        out = []
        for t in tokens:
            pos = st["n"]
            x = W["embed"][int(t)] * cfg["embedding"]["scale"]
            trail = []
            for i, spec in enumerate(cfg["layers"]):
                key = f"l{i}"
                h = layer_norm(x, W[key + ".norm1"], W[key + ".norm1.b"], eps)
                if spec["type"] == "mamba2":
                    x = x + ssm_token(W, key, spec["mixer"], h, st["mem"][i], eps)
                elif spec["type"] == "attention":
                    st["mem"][i].append(attention_kv(W, key, spec["mixer"], h, pos))
                    x = x + attention_token(W, key, spec["mixer"], h, pos, st["mem"][i])
                else:
                    raise ValueError(spec["type"])
                if spec.get("mlp") is not None:
                    x = x + relu2_ff(W, key, layer_norm(x, W[key + ".norm2"], W[key + ".norm2.b"], eps))
                trail.append(x.copy())
            if residuals is not None:
                residuals.append(np.stack(trail))
            xn = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
            out.append(soft_cap(W["embed"] @ xn, cfg.get("logit_softcap")))
            st["n"] += 1
        return np.stack(out)

    def drop(self, seq):
        self.seqs.pop(seq, None)


# ---- small random models for the tests ---------------------------------------------------------------------------------------


def bf16_round(a):
    u = np.asarray(a, dtype=np.float32).view(np.uint32)
    return (((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(np.float32)


def ssm_mixer(heads=4, vdim=8, state=8, groups=2, norm_groups=2, conv=3):
    return {"type": "mamba2", "mixer": {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state,
                                         "vdim": vdim}}


def attn_mixer(heads=4, kv_heads=2, dim=16, vdim=8, size=6, pool=3, dims=None, base=10000.0, scaling="default", scale=None):
    dims = dim if dims is None else dims
    if scaling == "default":
        scaling = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    return {"type": "attention", "mixer": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"pool": pool, "size": size},
                                           "rot": {"base": base, "dims": dims, "scaling": scaling},
                                           "scale": scale if scale is not None else dim ** -0.5, "vdim": vdim}}


def layer(mix, ff=None):
    return dict(mix, mlp=({"ff": ff, "kind": "dense"} if ff else None))


def small_config(layers, width=32, vocab=61, eps=1e-5, embed_scale=3.0, softcap=12.0):
    return {"architecture": "Tibalorn", "embedding": {"scale": embed_scale}, "layers": layers, "logit_softcap": softcap,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_model(cfg: dict, seed: int = 0) -> dict:
    """name -> float32 array (bfloat16-representable values), shapes from the configuration"""
    rng = np.random.default_rng(seed)
    Wd, out = cfg["width"], {}

    def mat(name, o, i, gain=1.0):
        out[name] = bf16_round(rng.standard_normal((o, i)) * gain / math.sqrt(i))

    def vec(name, n, centre=0.0, spread=0.1):
        out[name] = bf16_round(centre + rng.standard_normal(n) * spread)

    out["embed"] = bf16_round(rng.standard_normal((cfg["vocab"], Wd)) * 0.5)
    for i, spec in enumerate(cfg["layers"]):
        k, m = f"l{i}", spec["mixer"]
        vec(k + ".norm1", Wd, 1.0); vec(k + ".norm1.b", Wd)
        if spec["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            mat(k + ".mix.in", 2 * inner + 2 * gn + m["heads"], Wd)
            out[k + ".mix.conv"] = bf16_round(rng.standard_normal((inner + 2 * gn, m["conv"])) * 0.5)
            vec(k + ".mix.conv.b", inner + 2 * gn)
            vec(k + ".mix.dt_bias", m["heads"], -1.0, 0.5)
            out[k + ".mix.A_log"] = bf16_round(np.log(rng.uniform(0.3, 4.0, size=m["heads"])))
            vec(k + ".mix.D", m["heads"], 1.0, 0.3)
            vec(k + ".mix.norm", inner, 1.0)
            mat(k + ".mix.o", Wd, inner)
        else:
            H, G, dim, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(k + ".mix.q", H * dim, Wd, 2.0); vec(k + ".mix.q.b", H * dim, 0.0, 0.3)
            mat(k + ".mix.k", G * dim, Wd, 2.0); vec(k + ".mix.k.b", G * dim, 0.0, 0.3)
            mat(k + ".mix.v", G * vd, Wd); vec(k + ".mix.v.b", G * vd, 0.0, 0.3)
            vec(k + ".mix.temp", H, 1.0, 0.3); vec(k + ".mix.sink", H, 0.0, 1.0)
            mat(k + ".mix.g", H * vd, Wd); mat(k + ".mix.o", Wd, H * vd)
        if spec.get("mlp") is not None:
            vec(k + ".norm2", Wd, 1.0); vec(k + ".norm2.b", Wd)
            mat(k + ".mlp.up", spec["mlp"]["ff"], Wd); mat(k + ".mlp.down", Wd, spec["mlp"]["ff"])
    vec("final.norm", Wd, 1.0); vec("final.norm.b", Wd)
    return out
