"""Token-mixer combinators.  KParallelMixer runs two injected mixers side by side on the same input and returns half the sum of
their outputs, each first RMS-normed over the model width with its own plain weight:

    y = 0.5 * (rms(left(h)) * w_left + rms(right(h)) * w_right)

All input projections of both children are ONE GEMM (their weights are concatenated at load; the children read their columns of
its fp32 output), and with the fusion hooks of the decoder layer the combination, the layer's post-norm and the residual add are
one launch (`ktx_rms_combine`)."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule


class KParallelMixer(BaseInjectedModule):
    SUPPORTS_FUSION = True

    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        object.__setattr__(self, "eps", orig_module.eps)
        object.__setattr__(self, "w", {})

    def load(self):
        left, right = self.orig_module.left, self.orig_module.right
        for child in (left, right):
            if not hasattr(child, "in_weight_names"):
                raise RuntimeError(f"{self.key}: {type(child).__name__} was not replaced by an injected mixer (check the optimize rules)")
            child.load()
        ld, dev = self.gguf_loader, torch.device(self.device)
        self.w["in"] = torch.cat([left.w[n] for n, _ in left.in_weight_names()] + [right.w[n] for n, _ in right.in_weight_names()]).contiguous()
        self.w["right_base"] = sum(r for _, r in left.in_weight_names())
        self.w["left_out"] = ld.load_tensor(self.key + ".left.out", device=dev).to(torch.float32).contiguous()
        self.w["right_out"] = ld.load_tensor(self.key + ".right.out", device=dev).to(torch.float32).contiguous()

    def forward(self, h: torch.Tensor, batch, cache, post_norm=None, residual: torch.Tensor | None = None):
        """h fp32 [T, width].  Without hooks: the combined output fp32 [T, width].  With post_norm (a KResidualRMSNorm) and residual:
        residual += post_norm(combined), in place, returned."""
        from ktransformers_amd._native_seq import dense_gemm, rms_combine
        left, right = self.orig_module.left, self.orig_module.right
        proj = dense_gemm(h, self.w["in"])
        yl = left(h, batch, cache, proj=proj, q_off=0, k_off=left.heads * left.dim)
        yr = right(h, batch, cache, proj=proj, base=self.w["right_base"])
        if post_norm is not None and residual is not None:
            return rms_combine(yl, post_norm.weight_f32, self.eps, one_plus=post_norm.one_plus, residual=residual, y2=yr,
                               w1=self.w["left_out"], w2=self.w["right_out"])
        return rms_combine(yl, None, self.eps, y2=yr, w1=self.w["left_out"], w2=self.w["right_out"])
