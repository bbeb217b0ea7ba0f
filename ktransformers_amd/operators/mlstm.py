"""mLSTM (matrix-memory LSTM) mixer — an injected recurrent operator whose per-sequence state lives in the slots of a KHybridCache
(models/custom_cache.py) instead of a key / value cache:

    q = W_q h dim^-1/2, k = W_k h, v = W_v h per head; log gates i = cap tanh((W_i h + b_i) / cap),
    f = logsigmoid(cap tanh((W_f h + b_f) / cap)); with a running maximum m (0 at the start):
    m' = max(f + m, i), S' = e^(f + m - m') S + e^(i - m') k v^T, n' likewise with k,
    o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6); per-head unit RMS, weight, sigmoid(W_g h) gate, W_o.

State, gates and exponentials are fp32 (include/ktx_seq.h: `ktx_mlstm_forward` walks each request's new tokens in order, from the
slot's state or from zero at position 0; `ktx_mlstm_gate_norm` is the output norm and gate).  gate_cap and eps are constructor
arguments."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KMLSTMMixer(BaseInjectedModule):
    IN_ORDER = ("q", "k", "v", "g", "i", "f")

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("heads", "dim", "vdim", "gate_cap", "eps", "denom_eps", "layer_idx", "width"):
            object.__setattr__(self, name, getattr(o, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_cfg", None)

    def in_weight_names(self):
        N, D, V = self.heads, self.dim, self.vdim
        return [("q", N * D), ("k", N * D), ("v", N * V), ("g", N * V), ("i", N), ("f", N)]

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        for n, rows in self.in_weight_names():
            self.w[n] = ld.load_tensor(f"{self.key}.{n}", device=dev).to(cd).contiguous()
            if tuple(self.w[n].shape) != (rows, self.width):
                raise ValueError(f"{self.key}.{n}: shape {tuple(self.w[n].shape)} does not fit [{rows}, {self.width}]")
        self.w["o"] = ld.load_tensor(self.key + ".o", device=dev).to(cd).contiguous()
        for n in ("norm", "i.b", "f.b"):
            self.w[n] = ld.load_tensor(f"{self.key}.{n}", device=dev).to(torch.float32).contiguous()

    def forward(self, h: torch.Tensor, batch, cache, proj: torch.Tensor | None = None, base: int = 0):
        """proj: fp32 [T, *] holding this mixer's input projections from column `base` in IN_ORDER (computed here from h when not
        given).  Returns W_o(...) as fp32 [T, width]; the slot states of the batch's requests advance in place."""
        from ktransformers_amd._native_seq import dense_gemm, mlstm_config, mlstm_forward, mlstm_gate_norm
        if self._cfg is None:
            object.__setattr__(self, "_cfg", mlstm_config(self.heads, self.dim, self.vdim, self.gate_cap, self.eps, self.denom_eps))
        if proj is None:
            if "in" not in self.w:       # used on its own: all input projections as one product
                self.w["in"] = torch.cat([self.w[n] for n in self.IN_ORDER]).contiguous()
            proj, base = dense_gemm(h, self.w["in"]), 0
        offs, c = {}, base
        for n, rows in self.in_weight_names():
            offs[n] = c
            c += rows
        li = self.layer_idx
        o_raw = mlstm_forward(self._cfg, proj, offs, self.w["i.b"], self.w["f.b"], batch.q_indptr, batch.pos0, batch.slot,
                              cache.S[li], cache.n[li], cache.m[li], max_q_len=batch.max_q_len)
        o = mlstm_gate_norm(self._cfg, o_raw, proj, offs["g"], self.w["norm"], self.compute_dtype)
        return dense_gemm(o, self.w["o"])
