"""Sigmoid-weighted grouped-query attention with head mixing over a paged key cache — an injected operator beside the MLA ones
(operators/attention.py, balance_serve_attention.py), for designs whose attention is not a softmax:

    q = W_q h, k = W_k h (kv_heads <= heads), the VALUES ARE THE KEYS as projected (no W_v);
    q, k RMS-normed per head with a weight shared by the heads; q times a temperature 1 + c ln(floor((p + 1) / e) + 1);
    score(i, j) = scale q_i . k_j - slope_h (i - j),  slope_h = 2^(-span (h + 1) / heads);
    weight = sigmoid(score + bias_h) for j <= i, NOT normalised over keys; weights mixed across heads by a [heads, heads] matrix;
    head h applies its mixed weights to the rows of its own key head; W_o on the concatenated heads.

Every constant above (scale, c, e, span, eps) is a constructor argument.  The arithmetic is include/ktx_seq.h: `ktx_sigattn_prep`
(norms, temperature, cache append: the cache keeps the un-normed key row once — it serves as key and value — plus 1 / rms per row,
and the key norm's weight is folded into the query) and `ktx_sigattn_forward`.  Batching contract: the flattened tokens of a
ForwardBatch (models/custom_cache.py), the layer's key cache taken from the KHybridCache."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KSigmoidTalkAttention(BaseInjectedModule):
    TARGET_WORKGROUPS = 1024

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("heads", "kv_heads", "dim", "scale", "temp_coef", "temp_every", "slope_span", "eps", "layer_idx", "width"):
            object.__setattr__(self, name, getattr(o, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "_cfg", {})
        object.__setattr__(self, "w", {})

    def in_weight_names(self):
        """(suffix, rows) of the input projections, in the order their outputs are laid out."""
        return [("q", self.heads * self.dim), ("k", self.kv_heads * self.dim)]

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        f32 = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(torch.float32).contiguous()
        self.w.update(q=ld.load_tensor(self.key + ".q", device=dev).to(cd).contiguous(),
                      k=ld.load_tensor(self.key + ".k", device=dev).to(cd).contiguous(),
                      o=ld.load_tensor(self.key + ".o", device=dev).to(cd).contiguous(),
                      q_norm=f32("q.norm"), k_norm=f32("k.norm"), talk=f32("talk"), pb=f32("pb"))
        H, G, D = self.heads, self.kv_heads, self.dim
        if tuple(self.w["q"].shape) != (H * D, self.width) or tuple(self.w["k"].shape) != (G * D, self.width) or \
                tuple(self.w["o"].shape) != (self.width, H * D) or tuple(self.w["talk"].shape) != (H, H):
            raise ValueError(f"{self.key}: tensor shapes do not fit heads={H} kv_heads={G} dim={D} width={self.width}")

    def _config(self, cache):
        from ktransformers_amd._native_seq import sigattn_config
        k = (cache.page_size, cache.dtype)
        if k not in self._cfg:
            self._cfg[k] = sigattn_config(self.heads, self.kv_heads, self.dim, self.scale, self.temp_coef, self.temp_every,
                                          self.slope_span, cache.page_size, cache.dtype)
        return self._cfg[k]

    def forward(self, h: torch.Tensor, batch, cache, proj: torch.Tensor | None = None, q_off: int = 0, k_off: int | None = None):
        """h: fp32 [T, width] (read only when `proj` is not given); proj: fp32 [T, *] holding W_q h at q_off and W_k h at k_off.
        Returns W_o(attention) as fp32 [T, width]."""
        from ktransformers_amd._native_seq import dense_gemm, sigattn_forward, sigattn_prefill, sigattn_prefill_eligible, sigattn_prep
        if proj is None:
            if "qk" not in self.w:       # used on its own: the two input projections as one product
                self.w["qk"] = torch.cat([self.w["q"], self.w["k"]]).contiguous()
            proj = dense_gemm(h, self.w["qk"])
            q_off, k_off = 0, self.heads * self.dim
        cfg = self._config(cache)
        kc, kinv = cache.k_caches[self.layer_idx], cache.k_inv[self.layer_idx]
        q = sigattn_prep(cfg, proj, q_off, k_off, self.w["q_norm"], self.w["k_norm"], self.eps, batch.positions, batch.cache_loc, kc, kinv)
        if self.compute_dtype == torch.bfloat16 and sigattn_prefill_eligible(cfg):
            # matrix-core kernel: tiles of 16 query rows x key ranges, enough workgroups to fill the chip
            tiles = batch.B * ((batch.max_q_len + 15) // 16)
            nsplit = max(1, min(self.TARGET_WORKGROUPS // max(tiles, 1), (batch.max_kv_len + 31) // 32))
            a = sigattn_prefill(cfg, q, kc, kinv, batch.q_indptr, batch.pos0, batch.page_indptr, batch.page_indices, self.w["pb"],
                                self.w["talk"], batch.max_q_len, nsplit=nsplit)
            return dense_gemm(a, self.w["o"])
        a = sigattn_forward(cfg, q, kc, kinv, batch.tok_req, batch.positions, batch.page_indptr, batch.page_indices, self.w["pb"],
                            self.w["talk"], nsplit=batch.nsplit, out_dtype=self.compute_dtype)
        return dense_gemm(a, self.w["o"])
