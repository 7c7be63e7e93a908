"""Command line of the package: `python -m exllamav2_amd <command>`.

  generate  --model DIR --tokens "1,2,3" [--tokens ...] --max-new-tokens N [--temperature T --top-k K --top-p P --seed S]
            token-id prompts in, generated token ids out (one line per prompt); greedy unless a temperature is given
  trace     --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
            replays steps read from standard input, one JSON object a line
            {"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}], "end": [ids]}
            through Engine.step; writes OUT/<n>.f32 (little-endian fp32 [wanted, vocab]) for steps that want logits and prints
            "done <n>" after every step.  Nothing is sampled.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def _ensure_built(model_dir: str):
    """First use in a fresh checkout: compile in-tree what the model's architecture needs -- the subset library for the
    unquantized layer stacks, the whole library for the quantized Llama family.  A library that is already there is used as it is."""
    from . import _lib, build
    from .architectures import needs_whole_library
    if os.path.exists(_lib.HIP_LIB_PATH):
        return
    if needs_whole_library(model_dir):
        print("building the HIP library (first use) ...", file=sys.stderr, flush=True)
        build.build(verbose=False)
    elif not os.path.exists(_lib.HIP_DENSE_LIB_PATH):
        print("building the dense-model subset of the HIP library (first use) ...", file=sys.stderr, flush=True)
        build.build_dense(verbose=False)


def _dtype(name):
    import torch
    return {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16, None: None}[name]


def cmd_generate(a) -> int:
    _ensure_built(a.model)
    from .architectures import load_model
    from .engine import Engine, Generator
    model = load_model(a.model, device=a.device, dtype=_dtype(a.dtype))
    prompts = [[int(t) for t in s.replace(" ", "").split(",") if t] for s in a.tokens]
    need = sum(len(p) + a.max_new_tokens for p in prompts)
    eng = Engine(model, max_tokens=min(need, a.max_tokens) if a.max_tokens else need, max_seqs=a.max_seqs)
    out = Generator(eng, chunk=a.chunk).generate(prompts, a.max_new_tokens, temperature=a.temperature, top_k=a.top_k, top_p=a.top_p,
                                                 seed=a.seed)
    for toks in out:
        print(",".join(str(t) for t in toks))
    return 0


def cmd_trace(a) -> int:
    import torch
    if a.dtype not in ("bfloat16", "float32"):
        print("trace: --dtype is bfloat16 or float32", file=sys.stderr)
        return 2
    _ensure_built(a.model)
    from .architectures import load_model
    from .engine import Engine
    model = load_model(a.model, device=a.device, dtype=_dtype(a.dtype))
    if not hasattr(model, "step"):
        print("trace: this architecture has no step() forward", file=sys.stderr)
        return 2
    eng = Engine(model, max_tokens=a.max_tokens, max_seqs=a.max_seqs)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in step.get("entries", [])]
        logits = eng.step(entries, step.get("end", []))
        if logits is not None:
            data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{step['step']}.f32.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
        print(f"done {step['step']}", flush=True)
    return 0


def main(argv=None) -> int:
    p = argparse.ArgumentParser(prog="exllamav2_amd")
    sub = p.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate token ids from token-id prompts")
    g.add_argument("--model", required=True)
    g.add_argument("--tokens", action="append", required=True, help="a prompt as comma-separated token ids (repeatable)")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--dtype", default=None, choices=["bfloat16", "float32", "float16"])
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=1)
    g.add_argument("--top-p", type=float, default=0.0)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--chunk", type=int, default=512, help="largest portion of a prompt per step")
    g.add_argument("--max-tokens", type=int, default=0, help="cache pool size in tokens (default: what the prompts need)")
    g.add_argument("--max-seqs", type=int, default=4)
    g.add_argument("--device", default="cuda:0")
    g.set_defaults(fn=cmd_generate)
    t = sub.add_parser("trace", help="replay a step trace from standard input and write the wanted logits")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", default="bfloat16")
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True)
    t.add_argument("--max-seqs", type=int, default=4)
    t.add_argument("--device", default="cuda:0")
    t.set_defaults(fn=cmd_trace)
    a = p.parse_args(argv)
    return a.fn(a)


if __name__ == "__main__":
    sys.exit(main())
