"""Plain float64 restatement of the layer-stack models (exllamav2_amd/layered.py) -- TEST INFRASTRUCTURE ONLY.

One function per mechanism, written from the equations, token by token where that is the clearest form; nothing here is shared
with the product path (no absorbed projections, no pages, no batching: a sequence is a python list and its cache two lists).

Notation: h = a sublayer's input (the residual stream x itself: the layers are post-norm), W x with W stored [out, in].
    layer:    x <- N1(alpha x + mixer(x));  x <- N2(alpha x + ff(x));  N(v) = v / sqrt(mean(v^2) + eps) * (1 + w)
    latent attention, per token at position p:
        c_q = rms(W_dq h) * w_dq;  q = W_uq c_q, per head [dim unrotated | rot_dim rotated]
        d = W_dkv h;  c = rms(d[:kv_rank]) * w_dkv;  k_r = rot(d[kv_rank:], p)             (c and k_r are what a cache keeps)
        head i: k_i(j) = W_uk_i c_j,  v_i(j) = W_uv_i c_j,
                s_ij = (q_i[:dim] . k_i(j) + rot(q_i[dim:], p) . k_r(j)) * scale   for  0 <= p - j < window
                o_i = sum_j softmax_j(s_ij) v_i(j)
        out = W_o (concat_i o_i * sigmoid(W_g h))
        rot: the first `dims` values in pairs (2i, 2i+1): (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i/dims)
        kv_from = j: c and k_r are layer j's
    dense ff: W_down(silu(W_gate h) * W_up h)
    moe ff:   s = softmax(W_router h) over experts + identity outputs; chosen = top-k of (s + correction);
              weight_e = s_e / (sum of chosen s + 1e-20) * route_scale;
              expert: g = min(W_gate h, L), u = clamp(W_up h, -L, L), W_down(g sigmoid(1.702 g) (u + 1));
              the last `identity` outputs return h itself
    logits = W_head N_final(x)
"""
from __future__ import annotations

import math

import numpy as np


def rms(v: np.ndarray, eps: float) -> np.ndarray:
    return v / math.sqrt(float(np.mean(v * v)) + eps)


def post_norm(v: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return rms(v, eps) * (1.0 + w)


def rotate(vec: np.ndarray, pos: int, base: float, dims: int) -> np.ndarray:
    out = vec.copy()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        u, v = vec[2 * i], vec[2 * i + 1]
        out[2 * i] = u * math.cos(a) - v * math.sin(a)
        out[2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def softmax(z: np.ndarray) -> np.ndarray:
    e = np.exp(z - z.max())
    return e / e.sum()


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def latent_kv(W, key, m, h, pos, eps):
    """what the cache keeps for one token: (c, k_r)"""
    d = W[key + ".mix.dkv"] @ h
    R = m["kv_rank"]
    c = rms(d[:R], eps) * W[key + ".mix.dkv.norm"]
    return c, rotate(d[R:], pos, m["rot"]["base"], m["rot"]["dims"])


def latent_attention(W, key, m, h, pos, kv, eps):
    """kv: list over positions 0..pos of (c, k_r) (this token's included)"""
    H, dim, rd, vd = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms(W[key + ".mix.dq"] @ h, eps) * W[key + ".mix.dq.norm"]
    q = (W[key + ".mix.uq"] @ cq).reshape(H, dim + rd)
    lo = max(0, pos - m["mask"]["size"] + 1)
    heads = []
    for i in range(H):
        uk = W[key + ".mix.uk"][i * dim:(i + 1) * dim]
        uv = W[key + ".mix.uv"][i * vd:(i + 1) * vd]
        qr = rotate(q[i, dim:], pos, m["rot"]["base"], m["rot"]["dims"])
        s = np.array([(q[i, :dim] @ (uk @ kv[j][0]) + qr @ kv[j][1]) * m["scale"] for j in range(lo, pos + 1)])
        p = softmax(s)
        heads.append(sum(p[j - lo] * (uv @ kv[j][0]) for j in range(lo, pos + 1)))
    o = np.concatenate(heads) * sigmoid(W[key + ".mix.g"] @ h)
    return W[key + ".mix.o"] @ o


def dense_ff(W, key, h):
    g = W[key + ".mlp.gate"] @ h
    return W[key + ".mlp.down"] @ (g * sigmoid(g) * (W[key + ".mlp.up"] @ h))


def route(W, key, r, h):
    """(chosen expert ids, their weights)"""
    s = softmax(W[key + ".mlp.router"] @ h)
    choice = s + W[key + ".mlp.correction"]
    ids = sorted(range(len(s)), key=lambda e: (-choice[e], e))[:r["top"]]
    chosen = np.array([s[e] for e in ids])
    return ids, chosen / (chosen.sum() + 1e-20) * r["scale"]


def expert(W, key, e, limit, h):
    g = np.minimum(W[f"{key}.mlp.e{e}.gate"] @ h, limit)
    u = np.clip(W[f"{key}.mlp.e{e}.up"] @ h, -limit, limit)
    return W[f"{key}.mlp.e{e}.down"] @ (g * sigmoid(1.702 * g) * (u + 1.0))


def moe_ff(W, key, ms, h):
    r = ms["router"]
    ids, wts = route(W, key, r, h)
    y = np.zeros_like(h)
    for e, w in zip(ids, wts):
        y += w * (h if e >= r["experts"] else expert(W, key, e, ms["expert"]["limit"], h))
    return y


class Oracle:
    """A model and its sequences' caches; feed(seq, tokens) returns the logits of every fed token"""

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = cfg
        self.W = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.kv = {}                                      # sequence -> {layer: [(c, k_r) per position]}

    def feed(self, seq, tokens, residuals=None):
        cfg, W = self.cfg, self.W
        eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
        store = self.kv.setdefault(seq, {i: [] for i, L in enumerate(cfg["layers"]) if "kv_from" not in L["mixer"]})
        out = []
        for t in tokens:
            pos = len(next(iter(store.values())))
            x = W["embed"][t] * cfg["embedding"]["scale"]
            for i, L in enumerate(cfg["layers"]):
                key, m = f"l{i}", L["mixer"]
                if m.get("kv_from") is None:
                    store[i].append(latent_kv(W, key, m, x, pos, eps))
                    kv = store[i]
                else:
                    kv = store[m["kv_from"]]
                x = post_norm(alpha * x + latent_attention(W, key, m, x, pos, kv, eps), W[key + ".norm1"], eps)
                ms = L.get("mlp")
                if ms is not None:
                    y = dense_ff(W, key, x) if ms["kind"] == "dense" else moe_ff(W, key, ms, x)
                    x = post_norm(alpha * x + y, W[key + ".norm2"], eps)
                if residuals is not None:
                    residuals.append(x.copy())
            out.append(W["head"] @ post_norm(x, W["final.norm"], eps))
        return np.array(out)

    def drop(self, seq):
        self.kv.pop(seq, None)


def random_model(cfg: dict, seed: int = 0, bf16: bool = True) -> dict:
    """random weights with the tensor names of the design, as float32 arrays whose values are exact in bfloat16 (so the bfloat16
    and float32 product paths and this oracle all start from the same numbers)"""
    rng = np.random.default_rng(seed)
    W = {}

    def mat(name, out, inp, gain=1.0):
        W[name] = rng.standard_normal((out, inp)) * gain / math.sqrt(inp)

    def vec(name, n, centre=0.0, spread=0.1):
        W[name] = centre + rng.standard_normal(n) * spread

    width = cfg["width"]
    W["embed"] = rng.standard_normal((cfg["vocab"], width)) / 3.0
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        H, dim, rd, vd, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        vec(k + ".norm1", width);
        mat(k + ".mix.dq", Q, width); vec(k + ".mix.dq.norm", Q, 1.0)
        mat(k + ".mix.uq", H * (dim + rd), Q, 2.0)
        if m.get("kv_from") is None:
            mat(k + ".mix.dkv", R + rd, width, 2.0); vec(k + ".mix.dkv.norm", R, 1.0)
        mat(k + ".mix.uk", H * dim, R, 2.0); mat(k + ".mix.uv", H * vd, R)
        mat(k + ".mix.g", H * vd, width); mat(k + ".mix.o", width, H * vd, 2.0)
        ms = L.get("mlp")
        if ms is None:
            continue
        vec(k + ".norm2", width)
        if ms["kind"] == "dense":
            mat(k + ".mlp.gate", ms["ff"], width, 2.0); mat(k + ".mlp.up", ms["ff"], width, 2.0); mat(k + ".mlp.down", width, ms["ff"], 2.0)
        else:
            r, ff = ms["router"], ms["expert"]["ff"]
            for e in range(r["experts"]):
                mat(f"{k}.mlp.e{e}.gate", ff, width, 3.0); mat(f"{k}.mlp.e{e}.up", ff, width, 3.0); mat(f"{k}.mlp.e{e}.down", width, ff, 2.0)
            mat(k + ".mlp.router", r["experts"] + r.get("identity", 0), width, 4.0)
            vec(k + ".mlp.correction", r["experts"] + r.get("identity", 0), 0.0, 0.05)
    vec("final.norm", width)
    mat("head", cfg["vocab"], width, 2.0)
    if bf16:
        for k, v in W.items():
            u = np.asarray(v, dtype=np.float32).view(np.uint32)
            u = ((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)
            W[k] = u.view(np.float32)
    return {k: np.asarray(v, dtype=np.float32) for k, v in W.items()}


def small_config(layers, width=64, vocab=96, eps=1e-5, alpha=2.0, embed_scale=4.0) -> dict:
    return {"architecture": "Benolix", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps},
            "postln_alpha": alpha, "vocab": vocab, "width": width}


def mixer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=32, q_rank=24, window=6, base=10000.0, dims=None, scale=None, kv_from=None):
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "mask": {"size": window}, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim if dims is None else dims}, "rot_dim": rot_dim,
         "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def layer(mix, mlp):
    return {"mixer": mix, "mlp": mlp, "type": "latent_attention"}


def dense(ff=48):
    return {"ff": ff, "kind": "dense"}


def moe(experts=4, identity=2, top=2, ff=24, limit=1.5, scale=1.5):
    return {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "identity": identity, "scale": scale, "top": top}}
