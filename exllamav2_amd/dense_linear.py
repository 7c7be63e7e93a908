"""Linear layers over unquantized weights (bfloat16 or float32, stored [out, in]) on the HIP library's dense kernels
(csrc/dense.hip), beside the quantized ExLlamaV2Linear.  No library GEMM: every row count goes to exl2_dense_linear."""
from __future__ import annotations

import torch


class DenseLinear:
    """y = epilogue(x . w^T).  `w` may hold several slabs ([slabs, out, in]): per-head projections run as one batched call,
    expert weights are picked per row (`w_sel`) or per group."""

    def __init__(self, ext, key: str, weight: torch.Tensor):
        if weight.dim() not in (2, 3):
            raise RuntimeError(f"{key}: a linear weight is [out, in] or [slabs, out, in]")
        self.ext, self.key = ext, key
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape[-2], weight.shape[-1]
        self.slabs = weight.shape[0] if weight.dim() == 3 else 1

    @property
    def dtype(self):
        return self.weight.dtype

    def forward(self, x: torch.Tensor, rows: int, out_dtype=None, out: torch.Tensor | None = None, aux=None, epi: int = 0,
                limit: float = 0.0, ldx: int | None = None, x_off: int = 0, aux_ld: int = 0, aux_off: int = 0, bias=None) -> torch.Tensor:
        """Plain call on the first `rows` rows of x (leading dimension ldx, first value at element x_off); bias fp32 [out] or None."""
        n, k = self.out_features, self.in_features
        if out is None:
            out = torch.empty((rows, n), dtype=out_dtype or self.dtype, device=self.weight.device)
        self.ext.dense_linear(x, self.weight, out, rows, n, k, ldx or x.shape[-1], k, out.shape[-1], aux=aux, ldaux=aux_ld,
                              epi=epi, limit=limit, x_off=x_off, aux_off=aux_off, bias=bias)
        return out

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()
