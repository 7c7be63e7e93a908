"""Latent attention (beside ExLlamaV2Attention): queries through a low-rank latent, keys and values from ONE cached latent per token
plus one rotated key part shared by all heads, a sliding window, a sigmoid output gate.

Per token the cache holds c = rms_norm(W_dkv h)[:kv_rank] * w and k_rot = rot(W_dkv h[kv_rank:], pos).  Head i's key is
[W_uk_i c | k_rot] and its value W_uv_i c, so the kernels never expand a cached token per head:
    q_abs_i = W_uk_i^T q_nope_i                          (batched dense linear over the heads)
    o_lat_i = sum_j softmax_j((q_abs_i . c_j + rot(q_rot_i) . k_rot_j) scale) c_j        (csrc/latent_attn.hip, window of `window` keys)
    o_i     = (W_uv_i o_lat_i) * sigmoid(W_g h)_i        (batched dense linear, gate in its epilogue)
A layer built with `kv_from = j` has no W_dkv and attends over layer j's cached rows with its own W_uk / W_uv.
Everything the design leaves open is a constructor parameter: head count and the four per-head sizes, ranks, window, rotary
base / dims, score scale."""
from __future__ import annotations

import os

import torch

from .dense_linear import DenseLinear


def rotary_inv_freq(base: float, dims: int, device) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2: made in double precision, handed to the kernels as fp32"""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).to(torch.float32).to(device)


class LatentAttention:
    KEYS_PER_SPLIT = int(os.environ.get("EXL2_LATENT_KEYS_PER_SPLIT", "64"))     # decoded tokens: keys per workgroup of the split-key launch

    def __init__(self, model, key: str, layer_idx: int, *, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, q_rank: int,
                 window: int, rot_base: float, rot_dims: int, scale: float, kv_from: int | None = None):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.kv_rank, self.q_rank, self.window, self.scale = kv_rank, q_rank, window, scale
        self.rot_base, self.rot_dims, self.kv_from = rot_base, rot_dims, kv_from
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError(f"{key}: rot dims {rot_dims} must be even and at most rot_dim {rot_dim}")

    @property
    def cache_row_width(self) -> int:
        return self.kv_rank + self.rot_dim

    def load(self, get):
        """`get(name)` returns the device tensor `<layer>.mix.<name>` in the model's operand dtype"""
        H, dim, rd, vd, R = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        width = self.model.width
        dq, g = get("dq"), get("g")
        parts = [dq] + ([get("dkv")] if self.kv_from is None else []) + [g]
        # one linear for everything that reads the layer input: [dq | dkv | g]
        self.front = DenseLinear(self.ext, self.key + ".front", torch.cat(parts, 0))
        self.off_dkv = dq.shape[0]
        self.off_g = self.front.out_features - g.shape[0]
        self.dq_norm = get("dq.norm").contiguous()
        self.dkv_norm = get("dkv.norm").contiguous() if self.kv_from is None else None
        self.uq = DenseLinear(self.ext, self.key + ".uq", get("uq"))
        uk, uv = get("uk"), get("uv")
        if tuple(dq.shape) != (self.q_rank, width) or tuple(self.uq.weight.shape) != (H * (dim + rd), self.q_rank) \
                or tuple(uk.shape) != (H * dim, R) or tuple(uv.shape) != (H * vd, R) or tuple(g.shape) != (H * vd, width):
            raise RuntimeError(f"{self.key}: tensor shapes do not match the mixer's sizes")
        # absorbed key projection: slab i = W_uk_i^T as an [out = kv_rank, in = dim] weight
        self.uk_t = DenseLinear(self.ext, self.key + ".uk_t", uk.view(H, dim, R).transpose(1, 2).contiguous())
        self.uv = DenseLinear(self.ext, self.key + ".uv", uv.view(H, vd, R).contiguous())
        self.o = DenseLinear(self.ext, self.key + ".o", get("o"))
        self.inv_freq = rotary_inv_freq(self.rot_base, self.rot_dims, self.model.device) if self.rot_dims else \
            torch.zeros((1,), dtype=torch.float32, device=self.model.device)
        return self

    def weight_bytes(self) -> int:
        return sum(l.weight_bytes() for l in (self.front, self.uq, self.uk_t, self.uv, self.o))

    def forward(self, xh: torch.Tensor, rows: int, batch, cache) -> torch.Tensor:
        """xh: the layer input in the operand dtype [rows, width]; returns the mixer's output, fp32 [rows, width]"""
        ext, m = self.ext, self.model
        H, dim, rd, vd, R = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        dt, dev = m.dtype, m.device
        ncat = self.front.out_features
        f = self.front.forward(xh, rows, out=m.buf("mix.f", (rows, ncat), torch.float32))     # [rows, dq | dkv | g] fp32
        cq = m.buf("mix.cq", (rows, self.q_rank), dt)
        ext.rms_rows(f, ncat, self.dq_norm, False, cq, self.q_rank, rows, self.q_rank, m.norm_eps)
        q = self.uq.forward(cq, rows, out=m.buf("mix.q", (rows, H * (dim + rd)), dt))
        pool = cache.pool
        rows_cache = cache.layer(self.layer_idx)
        table = batch.block_table
        if self.kv_from is None:
            ext.latent_append(f, ncat, self.dkv_norm, m.norm_eps, rows, R, rd, self.rot_dims, self.inv_freq, batch.row_seq,
                              batch.row_pos, table, pool.page_size, rows_cache, dkv_off=self.off_dkv)
        hs = dim + rd
        q_abs = m.buf("mix.q_abs", (rows, H, R), torch.float32)
        ext.dense_linear(q, self.uk_t.weight, q_abs, rows, R, dim, H * hs, dim, H * R, batch=H, sxb=hs, swb=R * dim, syb=R)
        o_lat = m.buf("mix.o_lat", (rows, H, R), dt)
        tiled = ext.latent_attn_tiles_supported(dt, R, rd) and (batch.tiles16 is not None or batch.tiles1 is not None)
        if tiled:
            # matrix-core kernels: portions of prompts as tiles of 16 positions x one head per wave, decoded tokens as one position x
            # 16 heads per wave with the keys split over workgroups
            common = (q, H * hs, hs, dim, q_abs, rows_cache, pool.page_size, batch.row_seq, batch.row_pos, table, o_lat)
            if batch.tiles16 is not None:
                row0, nrows, n = batch.tiles16
                ext.latent_attn_tiles(*common, row0, nrows, n, 16, H, R, rd, self.rot_dims, self.inv_freq, self.scale, self.window)
            if batch.tiles1 is not None:
                row0, n, max_pos = batch.tiles1
                keys = min(self.window, max_pos + 1)
                nsplit = max(1, min(32, -(-keys // self.KEYS_PER_SPLIT)))
                part_o = part_ml = None
                if nsplit > 1:
                    part_o = m.buf("mix.part_o", (rows, H, nsplit, R), torch.float32)
                    part_ml = m.buf("mix.part_ml", (rows, H, nsplit, 2), torch.float32)
                ext.latent_attn_tiles(*common, row0, None, n, 1, H, R, rd, self.rot_dims, self.inv_freq, self.scale, self.window,
                                      nsplit=nsplit, part_o=part_o, part_ml=part_ml)
        else:
            ext.latent_attn(q, H * hs, hs, dim, q_abs, rows_cache, pool.page_size, batch.row_seq, batch.row_pos, table, o_lat,
                            rows, H, R, rd, self.rot_dims, self.inv_freq, self.scale, self.window)
        og = m.buf("mix.og", (rows, H * vd), dt)
        ext.dense_linear(o_lat, self.uv.weight, og, rows, vd, R, H * R, R, H * vd, batch=H, sxb=R, swb=vd * R, syb=vd,
                         aux=f, ldaux=ncat, sauxb=vd, aux_off=self.off_g, epi=ext.EPI_MUL_SIGMOID_AUX)
        return self.o.forward(og, rows, out=m.buf("mix.y", (rows, m.width), torch.float32))
