"""Grouped-head attention with a sliding window, pooled blocks behind the window, a sink in the softmax and rotated values
(beside LatentAttention and the quantized ExLlamaV2Attention).

Per token at position p, with h the layer input:
    [q | k | v | g] = W h + bias                      one dense linear (g has no bias)
    q, k: the first rot_dims values of every head turned by p * f_i, amplitudes times `amp` (rotary_tables: plain frequencies, or
          blended between f_i and f_i / factor by a ramp for long contexts); v: all vdim values turned by p * base^(-2m / vdim)
    the cache keeps the turned k and v per token, and per block of `pool` tokens their mean (cache.PagedKV)
    head i (key / value head i // (heads / kv_heads)) sees the tokens 0 <= p - j < window and the blocks wholly in front of the window:
          weights exp(s_j) / (exp(sink_i) + sum exp(s)),  s_j = q_i . k_j * scale * temp_i
    out = W_o (turn_back(sum_j w_j v_j, p) * sigmoid(g))                       (csrc/window_attn.hip)
Everything the design leaves open is a constructor parameter: head counts, sizes, window, block size, rotary base / dims / scaling /
pair layout, score scale; sink, per-head temperature and gate are used when the checkpoint has them."""
from __future__ import annotations

import math

import torch

from .cache import PagedKV
from .dense_linear import DenseLinear


def rotary_tables(base: float, dims: int, scaling: dict | None, device):
    """(frequencies fp32 [dims / 2], amplitude): f_i = base^(-2i / dims); with `scaling` = {factor, original, fast, slow} the
    frequency of pair i is f_i / factor * r_i + f_i (1 - r_i), r_i a ramp from 0 to 1 between the pair that makes `fast` turns
    over `original` positions and the one that makes `slow` turns, and cos / sin are multiplied by 0.1 ln(factor) + 1.  Made in
    double precision, handed to the kernels as fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    amp = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])

        def pair_of(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device), amp


class WindowAttention:
    MAX_SPLIT = 16                                            # decoded tokens: workgroups that share one row's key list

    def __init__(self, model, key: str, layer_idx: int, *, heads: int, kv_heads: int, dim: int, vdim: int, window: int, pool: int,
                 rot_base: float, rot_dims: int, rot_scaling: dict | None, scale: float, rotate_values: bool = True,
                 interleaved: bool = False):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.window, self.pool, self.scale = window, pool, scale
        self.rot_base, self.rot_dims, self.rot_scaling = rot_base, rot_dims, rot_scaling
        self.rotate_values, self.interleaved = rotate_values, interleaved
        if heads % kv_heads or rot_dims > dim or rot_dims % 2 or (rotate_values and vdim % 2) or window <= 0 or pool < 0:
            raise ValueError(f"{key}: inconsistent attention sizes")
        self.kv_from = None
        self.tiles_ok = self.ext.window_attn_tiles_supported(model.dtype, dim, vdim) and (self.heads * vdim) % 4 == 0

    def load(self, get):
        """`get(name)` returns the device tensor `<layer>.mix.<name>` in the model's operand dtype"""
        H, G, dim, vd, width, f32 = self.heads, self.kv_heads, self.dim, self.vdim, self.model.width, torch.float32
        dev = self.model.device
        q, k, v, g = get("q"), get("k"), get("v"), get("g")
        if tuple(q.shape) != (H * dim, width) or tuple(k.shape) != (G * dim, width) or tuple(v.shape) != (G * vd, width) \
                or tuple(g.shape) != (H * vd, width):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        # one linear for everything that reads the layer input: [q | k | v | g]
        self.front = DenseLinear(self.ext, self.key + ".front", torch.cat([q, k, v, g], 0))
        self.front_bias = torch.cat([get("q.b").to(f32), get("k.b").to(f32), get("v.b").to(f32),
                                     torch.zeros((H * vd,), dtype=f32, device=dev)]).contiguous()
        self.off_k, self.off_v, self.off_g = H * dim, (H + G) * dim, (H + G) * dim + G * vd
        self.q_scale = (get("temp").to(f32) * self.scale).contiguous()
        self.sink = get("sink").to(f32).contiguous()
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        if self.q_scale.numel() != H or self.sink.numel() != H or tuple(self.o.weight.shape) != (width, H * vd):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        self.freq, self.amp = rotary_tables(self.rot_base, self.rot_dims, self.rot_scaling, dev) if self.rot_dims else \
            (torch.zeros((1,), dtype=f32, device=dev), 1.0)
        self.vfreq, _ = rotary_tables(self.rot_base, vd, None, dev)
        return self

    def weight_bytes(self) -> int:
        return self.front.weight_bytes() + self.o.weight_bytes()

    def make_state(self, pool, dtype):
        return PagedKV(pool, self.kv_heads, self.dim, self.vdim, self.pool, dtype)

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the normed layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m, f32 = self.ext, self.model, torch.float32
        H, G, dim, vd = self.heads, self.kv_heads, self.dim, self.vdim
        st, page = cache.layer(self.layer_idx), cache.pool.page_size
        ncat = self.front.out_features
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, ncat), f32), bias=self.front_bias)        # [q | k | v | g] fp32
        q = m.buf("attn.q", (rows, H * dim), m.dtype)
        ext.kv_rot_append(f, ncat, 0, self.off_k, self.off_v, q, self.q_scale, st.k, st.v, st.k_pool, st.v_pool, self.freq, self.amp,
                          self.rot_dims, self.vfreq, self.rotate_values, self.interleaved, batch.row_seq, batch.row_pos, batch.block_table,
                          page, self.pool, rows, H, G, dim, vd)
        o = m.buf("attn.o", (rows, H * vd), m.dtype)
        common = (q, st.k, st.v, st.k_pool, st.v_pool, self.sink, f, ncat, self.off_g, self.vfreq, self.rotate_values, self.interleaved,
                  batch.row_seq, batch.row_pos, batch.block_table, page, self.pool, o)
        if self.tiles_ok and (batch.prompt_tiles is not None or batch.tiles1 is not None):
            # matrix-core kernels: portions of prompts as tiles of <= 64 positions x one head per workgroup, decoded tokens as one
            # row x one key / value head per workgroup (its query heads share the pass over the keys)
            if batch.prompt_tiles is not None:
                row0, nrow, n, size = batch.prompt_tiles
                ext.window_attn_tiles(*common, (row0, nrow, n), size, H, G, dim, vd, self.window)
            if batch.tiles1 is not None:
                row0, n, max_pos = batch.tiles1
                # the longest key list among the rows: window tokens + pooled blocks; its steps of 128 entries go to up to 16 workgroups
                entries = min(self.window, max_pos + 1) + (max(0, max_pos - self.window + 1) // self.pool if self.pool else 0)
                nsplit = max(1, min(self.MAX_SPLIT, -(-entries // 128)))
                part_o = part_ml = None
                if nsplit > 1:
                    part_o = m.buf("attn.part_o", (rows, H, nsplit, vd), f32)
                    part_ml = m.buf("attn.part_ml", (rows, H, nsplit, 2), f32)
                ext.window_attn_tiles(*common, (row0, None, n), 1, H, G, dim, vd, self.window, nsplit=nsplit, part_o=part_o, part_ml=part_ml)
        else:
            ext.window_attn(*common, rows, H, G, dim, vd, self.window)
        return self.o.forward(o, rows, out=m.buf("mix.y", (rows, m.width), f32))
