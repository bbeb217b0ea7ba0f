"""Injected token embeddings.  KSinusoidEmbedding: x[t] = table[token] + s(position), the fixed sinusoid
s(p)[2i] = sin(p base^(-2i / width)), s(p)[2i + 1] = cos(p base^(-2i / width)), written as the fp32 residual stream
(include/ktx_seq.h `ktx_embed_sinpos`: the angle and its sine in fp64, one rounding).  `base` is a constructor argument."""
from __future__ import annotations

import torch

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KSinusoidEmbedding(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 base: float = 10000.0, **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "base", float(base))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        dev = torch.device(self.device)
        table = self.gguf_loader.load_tensor(self.key, device=dev).to(self.compute_dtype).contiguous()
        width = table.shape[1]
        i = torch.arange((width + 1) // 2, dtype=torch.float64)
        self.w.update(table=table, inv_freq=torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / width).to(dev))

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        from ktransformers_amd._native_seq import embed_sinpos
        return embed_sinpos(tokens.reshape(-1).to(torch.int32), positions.reshape(-1).to(torch.int32), self.w["table"], self.w["inv_freq"])


class KTableEmbedding(BaseInjectedModule):
    """x[t] = table[token] written as the fp32 residual stream (positions enter elsewhere, e.g. by rotation in the attention);
    include/ktx_seq.h `ktx_embed_sinpos` without its positional term."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})

    def load(self):
        self.w["table"] = self.gguf_loader.load_tensor(self.key, device=torch.device(self.device)).to(self.compute_dtype).contiguous()

    def forward(self, tokens: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        from ktransformers_amd._native_seq import embed_rows
        return embed_rows(tokens.reshape(-1).to(torch.int32), self.w["table"])


class KPassOffset(BaseInjectedModule):
    """What a block of layers that runs several times with the same weights adds to the residual stream in front of pass t:
    the embedding output again (every pass but the first) and a learned vector per pass, table[t] — one launch
    (include/ktx_hyb.h `ktx_rows_add`).  Checkpoint tensor: `<key>.step` [passes, width]."""

    def __init__(self, key: str, gguf_loader, config, orig_module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 table_suffix: str = ".step", **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "table_suffix", table_suffix)
        object.__setattr__(self, "w", {})

    def load(self):
        t = self.gguf_loader.load_tensor(self.key + self.table_suffix, device=torch.device(self.device)).to(torch.float32).contiguous()
        if t.dim() != 2 or t.shape[0] < self.orig_module.times:
            raise ValueError(f"{self.key}{self.table_suffix}: expected [passes >= {self.orig_module.times}, width], got {tuple(t.shape)}")
        self.w["step"] = t

    def forward(self, x: torch.Tensor, x0: torch.Tensor, t: int) -> torch.Tensor:
        from ktransformers_amd._native_hyb import rows_add
        return rows_add(x, x0 if t > 0 else None, self.w["step"][t])
