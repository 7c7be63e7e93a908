"""ExLlamaV2MLP (reference mlp.py:150-223 load/make_q_mlp, :318-361 forward)."""
from __future__ import annotations

import torch

from .ext import none_tensor
from .linear import ExLlamaV2Linear


class ExLlamaV2MLP:
    def __init__(self, model, key: str, layer_idx: int):
        cfg = model.config
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.gate_proj = ExLlamaV2Linear(self.ext, key + ".mlp.gate_proj", cfg.hidden_size, cfg.intermediate_size, model)
        self.up_proj = ExLlamaV2Linear(self.ext, key + ".mlp.up_proj", cfg.hidden_size, cfg.intermediate_size, model)
        self.down_proj = ExLlamaV2Linear(self.ext, key + ".mlp.down_proj", cfg.intermediate_size, cfg.hidden_size, model)
        self.q_handle = None

    def load(self, ck: dict):
        cfg, m = self.model.config, self.model
        for lin in (self.gate_proj, self.up_proj, self.down_proj):
            lin.load(ck[lin.key])
        self.post_attention_layernorm = ck[self.key + ".post_attention_layernorm"]
        self.q_handle = self.ext.make_q_mlp(                                     # mlp.py:204-223
            self.post_attention_layernorm, none_tensor, True, cfg.norm_eps,
            self.gate_proj.q_handle, self.up_proj.q_handle, self.down_proj.q_handle,
            m.temp_state, m.temp_a, m.temp_b, none_tensor, m.max_rows, False, True, none_tensor, none_tensor, False, False)
        return self

    def unload(self):
        if self.q_handle is not None:
            self.ext.free_q_mlp(self.q_handle)
            self.q_handle = None
        for lin in (self.gate_proj, self.up_proj, self.down_proj):
            lin.unload()

    def forward(self, hidden_states: torch.Tensor):
        """mlp.py:353: ext_c.q_mlp_forward_ in place, for every row count (<= 16 rows: the fused decode launches; above:
        row pre-pass + dequantize-into-MFMA GEMMs, csrc/modules.hip:exl2_q_mlp_forward)."""
        self.ext.q_mlp_forward_(self.q_handle, hidden_states)
        return hidden_states


class DenseGatedMLP:
    """Gated MLP over unquantized weights: W_down(silu(W_gate h) * (W_up h)) in three launches -- the activation and the product
    run in the up projection's epilogue (csrc/dense.hip).  Returns the sublayer's output in fp32; the residual step is the
    caller's (pre- or post-norm)."""

    def __init__(self, model, key: str, layer_idx: int):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx

    def load(self, get):
        from .dense_linear import DenseLinear
        self.gate = DenseLinear(self.ext, self.key + ".gate", get("gate"))
        self.up = DenseLinear(self.ext, self.key + ".up", get("up"))
        self.down = DenseLinear(self.ext, self.key + ".down", get("down"))
        return self

    def weight_bytes(self) -> int:
        return self.gate.weight_bytes() + self.up.weight_bytes() + self.down.weight_bytes()

    def forward(self, xh: torch.Tensor, rows: int):
        m, ff = self.model, self.gate.out_features
        g = self.gate.forward(xh, rows, out=m.buf("ff.g", (rows, ff), torch.float32))
        a = self.up.forward(xh, rows, out=m.buf("ff.a", (rows, ff), m.dtype), aux=g, aux_ld=ff, epi=self.ext.EPI_SILU_AUX_MUL)
        return self.down.forward(a, rows, out=m.buf("ff.y", (rows, m.width), torch.float32)), None


class DenseActMLP:
    """Two-matrix feed-forward over unquantized weights: W_down act(W_up h), the activation in the up projection's epilogue
    (csrc/dense.hip).  act: an epilogue code of the dense linear (default relu(z)^2)."""

    def __init__(self, model, key: str, layer_idx: int, act: int | None = None):
        self.model, self.ext, self.key, self.layer_idx = model, model.ext, key, layer_idx
        self.act = self.ext.EPI_RELU_SQUARED if act is None else act

    def load(self, get):
        from .dense_linear import DenseLinear
        self.up = DenseLinear(self.ext, self.key + ".up", get("up"))
        self.down = DenseLinear(self.ext, self.key + ".down", get("down"))
        if self.down.in_features != self.up.out_features:
            raise RuntimeError(f"{self.key}: up is {tuple(self.up.weight.shape)}, down is {tuple(self.down.weight.shape)}")
        return self

    def weight_bytes(self) -> int:
        return self.up.weight_bytes() + self.down.weight_bytes()

    def forward(self, xh: torch.Tensor, rows: int):
        m, ff = self.model, self.up.out_features
        a = self.up.forward(xh, rows, out=m.buf("ff.a", (rows, ff), m.dtype), epi=self.act)
        return self.down.forward(a, rows, out=m.buf("ff.y", (rows, m.width), torch.float32)), None
