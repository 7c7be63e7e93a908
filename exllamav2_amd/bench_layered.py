"""Prefill and decode throughput of a latent-attention / scored-MoE layer stack at layer sizes of real models (random weights),
beside the closest quantized model of the package (a Mixtral-style EXL2 stack) at the same width, expert width, expert count and
depth.  Used by `bench.py --design benolix`; one JSON object per size."""
from __future__ import annotations

import json
import time

import torch

SIZES = {
    # width, heads, dim, rot, vdim, kv_rank, q_rank, window, experts, identity, top, expert ff, dense ff, layers, vocab
    "w2048": dict(width=2048, heads=16, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=768, window=1024, experts=8, identity=2, top=2,
                  ff=5632, dense_ff=5632, layers=4, vocab=32000),
    "w4096": dict(width=4096, heads=32, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=1536, window=2048, experts=8, identity=2, top=2,
                  ff=14336, dense_ff=14336, layers=2, vocab=32000),
}


def layered_config(s: dict) -> dict:
    def mixer(kv_from=None):
        m = {"dim": s["dim"], "heads": s["heads"], "kv_rank": s["kv_rank"], "mask": {"size": s["window"]}, "q_rank": s["q_rank"],
             "rot": {"base": 10000.0, "dims": s["rot"]}, "rot_dim": s["rot"], "scale": (s["dim"] + s["rot"]) ** -0.5, "vdim": s["vdim"]}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return m
    moe = {"expert": {"ff": s["ff"], "limit": 7.0}, "kind": "moe",
           "router": {"experts": s["experts"], "identity": s["identity"], "scale": 1.0, "top": s["top"]}}
    layers = []
    for i in range(s["layers"]):
        layers.append({"type": "latent_attention", "mixer": mixer(None if i % 2 == 0 else i - 1),
                       "mlp": {"ff": s["dense_ff"], "kind": "dense"} if i == 0 else moe})
    return {"architecture": "Benolix", "embedding": {"scale": 1.0}, "layers": layers, "norm": {"eps": 1e-5}, "postln_alpha": 1.0,
            "vocab": s["vocab"], "width": s["width"]}


def random_tensors(cfg: dict, device, seed: int = 0) -> dict:
    g = torch.Generator(device=device).manual_seed(seed)
    T = {}

    def mat(name, out, inp):
        T[name] = (torch.randn((out, inp), device=device, generator=g) / inp ** 0.5).to(torch.bfloat16)

    def vec(name, n, centre):
        T[name] = (centre + 0.1 * torch.randn((n,), device=device, generator=g)).to(torch.bfloat16)

    w = cfg["width"]
    mat("embed", cfg["vocab"], 1); mat("head", cfg["vocab"], w); vec("final.norm", w, 0.0)
    T["embed"] = (torch.randn((cfg["vocab"], w), device=device, generator=g)).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        m, k = L["mixer"], f"l{i}"
        H, dim, rd, vd, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        vec(k + ".norm1", w, 0.0); vec(k + ".norm2", w, 0.0)
        mat(k + ".mix.dq", Q, w); vec(k + ".mix.dq.norm", Q, 1.0); mat(k + ".mix.uq", H * (dim + rd), Q)
        if "kv_from" not in m:
            mat(k + ".mix.dkv", R + rd, w); vec(k + ".mix.dkv.norm", R, 1.0)
        mat(k + ".mix.uk", H * dim, R); mat(k + ".mix.uv", H * vd, R); mat(k + ".mix.g", H * vd, w); mat(k + ".mix.o", w, H * vd)
        ms = L["mlp"]
        if ms["kind"] == "dense":
            mat(k + ".mlp.gate", ms["ff"], w); mat(k + ".mlp.up", ms["ff"], w); mat(k + ".mlp.down", w, ms["ff"])
        else:
            r = ms["router"]
            for e in range(r["experts"]):
                mat(f"{k}.mlp.e{e}.gate", ms["expert"]["ff"], w); mat(f"{k}.mlp.e{e}.up", ms["expert"]["ff"], w)
                mat(f"{k}.mlp.e{e}.down", w, ms["expert"]["ff"])
            mat(k + ".mlp.router", r["experts"] + r["identity"], w)
            T[k + ".mlp.correction"] = torch.zeros((r["experts"] + r["identity"],), device=device, dtype=torch.bfloat16)
    return T


def _timed(fn, reps: int):
    """seconds per call; the interpreter's cyclic collector is held off while the clock runs (a full collection of a process that has
    imported torch takes tens of milliseconds and would land in one of a few repetitions)"""
    import gc
    gc.collect()
    gc.disable()
    try:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps
    finally:
        gc.enable()


def bench_layered(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    from .config import LayeredConfig
    from .engine import Engine
    from .layered import LayeredModel
    s = SIZES[size]
    cfg = layered_config(s)
    model = LayeredModel(LayeredConfig.from_dict(cfg), device=device, dtype=torch.bfloat16).load(random_tensors(cfg, device))
    out = {"design": "benolix", "size": size, "layers": s["layers"], "weight_bytes_per_token": model.weight_bytes()}
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, s["vocab"], (prompt,), generator=g).tolist()
    eng = Engine(model, max_tokens=max(prompt, max(batches) * (ctx + decode_steps + 8)) + 256, max_seqs=max(4, max(batches)))
    eng.step([("warm", toks, [prompt - 1])], ["warm"])
    dt = _timed(lambda: eng.step([("p", toks, [prompt - 1])], ["p"]), 3)
    out["prefill_tokens_per_s"] = prompt / dt
    out["prefill_ms"] = dt * 1e3
    for b in batches:
        ids = [f"d{i}" for i in range(b)]
        eng.step([(r, toks[:ctx], []) for r in ids])
        step = lambda: eng.step([(r, [7], [0]) for r in ids])
        step()
        dt = _timed(step, decode_steps)
        out[f"decode_b{b}_tokens_per_s"] = b / dt
        out[f"decode_b{b}_ms_per_step"] = dt * 1e3
        for r in ids:
            eng.finish(r)
    return out


def bench_quantized_peer(size: str, device="cuda:0", prompt: int = 2048, ctx: int = 1024, decode_steps: int = 64, batches=(1, 4)) -> dict:
    """the package's Mixtral-style EXL2 stack (4.0 bpw) with the same width, expert width / count / top-k, depth and vocabulary"""
    from . import ExLlamaV2, ExLlamaV2Cache, ExLlamaV2Config, GreedyGraphDecoder
    from .synth import synth_checkpoint
    s = SIZES[size]
    out = {"design": "mixtral-exl2-4.0bpw", "size": size, "layers": s["layers"]}
    for b in batches:
        cfg = ExLlamaV2Config(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=s["layers"],
                              num_attention_heads=s["heads"], num_key_value_heads=max(1, s["heads"] // 4), head_dim=128,
                              vocab_size=s["vocab"], max_seq_len=4096, max_input_len=prompt, max_batch_size=1,
                              num_experts=s["experts"], num_experts_per_token=s["top"], arch="mixtral")
        ck = synth_checkpoint(cfg, device, recipe="4.0bpw", seed=0)
        model = ExLlamaV2(cfg, device=device).load(ck)
        g = torch.Generator().manual_seed(1)
        ids = torch.randint(0, s["vocab"], (1, prompt), generator=g)
        if b == batches[0]:
            cache = ExLlamaV2Cache(model, batch_size=1)
            model.forward(ids, cache)
            def pre():
                cache.current_seq_len = 0
                model.forward(ids, cache)
            dt = _timed(pre, 3)
            out["prefill_tokens_per_s"] = prompt / dt
            out["prefill_ms"] = dt * 1e3
            out["weight_bytes_per_token"] = model.weight_bytes()
            del cache
        cache = ExLlamaV2Cache(model, batch_size=b)
        dec = GreedyGraphDecoder(model, cache, batch_size=b).capture()
        dec.reset(torch.zeros((b,), dtype=torch.int32), ctx)
        dec.run(8)
        dec.reset(torch.zeros((b,), dtype=torch.int32), ctx)
        dt = _timed(lambda: dec.run(1), decode_steps)
        out[f"decode_b{b}_tokens_per_s"] = b / dt
        out[f"decode_b{b}_ms_per_step"] = dt * 1e3
        dec.free(); model.unload()
        del dec, cache, model, ck
        torch.cuda.empty_cache()
    return out


def run(sizes, device="cuda:0", peer: bool = True):
    for size in sizes:
        print(json.dumps(bench_layered(size, device)), flush=True)
        if peer:
            print(json.dumps(bench_quantized_peer(size, device)), flush=True)
