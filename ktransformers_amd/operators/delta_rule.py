"""Gated delta-rule mixer — an injected recurrent operator beside the mLSTM (operators/mlstm.py); its per-sequence state lives in the
slots of a KHybridCache (models/custom_cache.py): the memory S [heads, dim, vdim] and the last taps - 1 inputs of its convolutions.

    q = W_q h, k = W_k h (kv_heads x dim), v = W_v h (heads x vdim); head j reads q / k head j // (heads / kv_heads);
    each channel of q, k, v passes a causal convolution over time (`<key>.{q,k,v}.conv` [channels, taps], last column = now), then silu;
    q, k -> unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q also times dim^-1/2;
    beta = sigmoid(W_b h), g = exp(-exp(A_log) softplus(W_a h + dt_bias)) per head;
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
    per head o / rms(o) (eps) * norm (one weight per value entry, shared by the heads) * silu(W_g h);  W_o.

State, decays, steps, unit vectors and the output norm are fp32 in every number format (include/ktx_hyb.h: `ktx_delta_prep`,
`ktx_delta_forward`, `ktx_head_gate_norm`).  All input projections — and a rider's (operators/linear.py KLinearRider) — are ONE GEMM.
unit_eps and eps are constructor arguments."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule
from ktransformers_amd.operators.linear import merged_input_weight


class KGatedDeltaMixer(BaseInjectedModule):
    IN_ORDER = ("q", "k", "v", "g", "b", "a")

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("heads", "kv_heads", "dim", "vdim", "taps", "eps", "unit_eps", "width"):
            object.__setattr__(self, name, getattr(o, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_cfg", None)
        object.__setattr__(self, "_merged", {})

    def in_weight_names(self):
        H, G, D, V = self.heads, self.kv_heads, self.dim, self.vdim
        return [("q", G * D), ("k", G * D), ("v", H * V), ("g", H * V), ("b", H), ("a", H)]

    def state_spec(self) -> dict:
        return {"delta": (self.heads, self.dim, self.vdim), "conv": (2 * self.kv_heads * self.dim + self.heads * self.vdim, self.taps)}

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        for n, rows in self.in_weight_names():
            self.w[n] = ld.load_tensor(f"{self.key}.{n}", device=dev).to(cd).contiguous()
            if tuple(self.w[n].shape) != (rows, self.width):
                raise ValueError(f"{self.key}.{n}: shape {tuple(self.w[n].shape)} does not fit [{rows}, {self.width}]")
        self.w["o"] = ld.load_tensor(self.key + ".o", device=dev).to(cd).contiguous()
        f32 = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(torch.float32).contiguous()
        self.w["taps"] = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")]).contiguous()
        if self.w["taps"].shape[1] != self.taps:
            raise ValueError(f"{self.key}: convolutions of {self.w['taps'].shape[1]} taps, the config says {self.taps}")
        for n in ("norm", "A_log", "dt_bias"):
            self.w[n] = f32(n)

    def _input_weight(self, rider):
        k = id(rider) if rider is not None else None
        if k not in self._merged:
            self._merged[k] = merged_input_weight([self.w[n] for n in self.IN_ORDER], rider)
        return self._merged[k]

    def forward(self, h: torch.Tensor, batch, cache, cache_idx: int, rider=None):
        """h [T, width] in the compute type.  Returns (W_o(...) fp32 [T, width], the rider's product fp32 [T, rider rows] or None); the
        slot states of the batch's requests advance in place."""
        from ktransformers_amd._native_hyb import delta_config, delta_forward, delta_prep, head_gate_norm
        from ktransformers_amd._native_seq import dense_gemm
        if self._cfg is None:
            object.__setattr__(self, "_cfg", delta_config(self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.unit_eps))
        proj = dense_gemm(h, self._input_weight(rider))
        offs, c = {}, 0
        for n, rows in self.in_weight_names():
            offs[n] = c
            c += rows
        qkv, gb = delta_prep(self._cfg, proj, offs, self.w["taps"], self.w["A_log"], self.w["dt_bias"], batch, cache.conv[cache_idx])
        o_raw = delta_forward(self._cfg, qkv, gb, batch, cache.S[cache_idx])
        HV = self.heads * self.vdim
        o = head_gate_norm(o_raw, proj[:, offs["g"]:offs["g"] + HV], self.w["norm"], self.heads, self.vdim, self.eps, False, "silu",
                           out_dtype=self.compute_dtype)
        return dense_gemm(o, self.w["o"]), (proj[:, c:] if rider is not None else None)
