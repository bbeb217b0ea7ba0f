"""Sigmoid-routed mixture of GLU experts on an fp32 residual stream, any sizes, bf16 or fp32 — an injected operator beside the
quantised MoE operators (operators/experts.py, gate.py), which serve the DeepSeek / Mixtral families:

    s = sigmoid(W_router h) (fp32 accumulation and scores);  the `top` experts with the largest s;  weights = s_chosen / (sum of the
    chosen s + 1e-20) * scale;  expert e: W_down (silu(W_gate h) * (W_up h)), no biases;  out = sum of the weighted chosen experts
    + a shared expert of the same form that every token takes.

One input GEMM computes the router logits, the shared expert's gate | up and a rider's product (operators/linear.py KLinearRider).
The routed experts run as two grouped GEMMs over the (token, choice) pairs sorted by expert (include/ktx_hyb.h `ktx_moe_route`,
`ktx_moe_plan`, `ktx_grouped_gemm`); the weighted sum over a token's choices is left to the consumer's kernel (`ktx_gated_norm_add`
gathers the rows), so forward returns the pieces.  top, scale and the sum's eps are constructor arguments (read from the replaced
module).  Checkpoint tensors: `<key>.router` [experts, width], `<key>.e<i>.{gate,up,down}`, `<key>.shared.{gate,up,down}`."""
from __future__ import annotations

import torch
from torch import nn

from ktransformers_amd.operators.base_operator import BaseInjectedModule
from ktransformers_amd.operators.linear import merged_input_weight


class KSigmoidRoutedMoE(BaseInjectedModule):
    def __init__(self, key: str, gguf_loader, config, orig_module: nn.Module, prefill_device: str = "cuda", generate_device: str = "cuda",
                 **kwargs):
        BaseInjectedModule.__init__(self, key, gguf_loader, config, orig_module, prefill_device, generate_device, **kwargs)
        o = orig_module
        for name in ("experts", "top", "route_scale", "sum_eps", "ff", "shared_ff", "width"):
            object.__setattr__(self, name, getattr(o, name))
        object.__setattr__(self, "compute_dtype", getattr(config, "compute_dtype", torch.bfloat16))
        object.__setattr__(self, "w", {})
        object.__setattr__(self, "_merged", {})

    RETURNS_EXPERT_ROWS = True      # forward hands the routed experts' rows back un-summed (the consumer's kernel gathers them)

    def load(self):
        ld, dev, cd = self.gguf_loader, torch.device(self.device), self.compute_dtype
        get = lambda n: ld.load_tensor(f"{self.key}.{n}", device=dev).to(cd)
        E, F, W = self.experts, self.ff, self.width
        self.w["router"] = get("router").contiguous()
        # per expert [gate ; up] as one [2 ff, width] matrix, experts back to back
        self.w["gate_up"] = torch.stack([torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")]) for e in range(E)]).contiguous()
        self.w["down"] = torch.stack([get(f"e{e}.down") for e in range(E)]).contiguous()
        if tuple(self.w["gate_up"].shape) != (E, 2 * F, W) or tuple(self.w["down"].shape) != (E, W, F) or \
                tuple(self.w["router"].shape) != (E, W):
            raise ValueError(f"{self.key}: expert tensors do not fit experts={E} ff={F} width={W}")
        if self.shared_ff:
            self.w["shared_gate_up"] = torch.cat([get("shared.gate"), get("shared.up")]).contiguous()
            self.w["shared_down"] = get("shared.down").contiguous()
            if tuple(self.w["shared_gate_up"].shape) != (2 * self.shared_ff, W):
                raise ValueError(f"{self.key}.shared: tensors do not fit ff={self.shared_ff}")

    def forward(self, h: torch.Tensor, rider=None):
        """h [T, width] in the compute type -> (shared expert's output fp32 [T, width] or None, the rider's product or None,
        expert_rows fp32 [T * top, width] in sorted order, pair_pos int32 [T * top], topk_w fp32 [T, top])."""
        from ktransformers_amd._native_hyb import GEMV_MAX_ROWS, WIDE_MIN_ROWS_PER_EXPERT, expert_gemm, moe_plan, moe_route, silu_mul_rows
        from ktransformers_amd._native_seq import dense_gemm
        k = id(rider) if rider is not None else None
        if k not in self._merged:
            own = [self.w["router"]] + ([self.w["shared_gate_up"]] if self.shared_ff else [])
            self._merged[k] = merged_input_weight(own, rider)
        E, SF = self.experts, self.shared_ff or 0
        proj = dense_gemm(h, self._merged[k])
        idx, wts = moe_route(proj[:, :E], self.top, self.route_scale, self.sum_eps)
        wide = self.compute_dtype == torch.bfloat16 and h.shape[0] * self.top >= WIDE_MIN_ROWS_PER_EXPERT * E
        plan = moe_plan(idx, E, wide=wide)
        if plan.pairs <= GEMV_MAX_ROWS:      # decode steps: the weights stream once per pair, the activation in the same launch
            act = expert_gemm(h, self.w["gate_up"], plan, gather=True, out_dtype=self.compute_dtype, glu=True)
        else:
            act = silu_mul_rows(expert_gemm(h, self.w["gate_up"], plan, gather=True), out_dtype=self.compute_dtype)
        rows = expert_gemm(act, self.w["down"], plan, gather=False)
        shared = None
        if SF:
            shared = dense_gemm(silu_mul_rows(proj[:, E:E + 2 * SF], out_dtype=self.compute_dtype), self.w["shared_down"])
        return shared, (proj[:, E + 2 * SF:] if rider is not None else None), rows, plan.pair_pos, wts
