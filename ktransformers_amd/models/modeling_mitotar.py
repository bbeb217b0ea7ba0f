"""Module skeleton of Mitotar — a post-norm decoder with an fp32 residual stream whose layers mix tokens with two mixers side
by side (sigmoid attention with head mixing whose values are its keys, and an mLSTM) and a dense GELU feed-forward.

Like the other skeletons of this package it only holds the structure the optimize rules inject into (optimize_rules/Mitotar.yaml)
and the glue (the layer loop); every module that does arithmetic is a leaf that raises until an operator replaces it.  Module
paths equal the checkpoint's tensor prefixes, so an injected operator finds its tensors under its own key:

    embed | l<i>.mix.{left,right} | l<i>.norm1 | l<i>.mlp | l<i>.norm2 | final.norm | head

config.json: {"architecture": "Mitotar", "width", "vocab", "norm": {"eps"}, "layers": [{"type": "parallel", "mixer": {"left":
{"heads", "kv_heads", "dim", "vdim", "scale", "q_temp": {"coef", "every"}}, "right": {"heads", "dim", "vdim", "gate_cap"}},
"mlp": {"kind": "dense", "ff"} | null}, ...]}.  Sizes and the constants listed there come from the file; what the design fixes
is a constant here."""
from __future__ import annotations

import json
import os
from types import SimpleNamespace

import torch
from torch import nn

from ktransformers_amd.models.modeling_deepseek import _Leaf

# fixed by the design
DISTANCE_SLOPE_SPAN = 8.0      # slope_h = 2^(-8 (h + 1) / heads)
SINUSOID_BASE = 10000.0
MLSTM_DENOM_EPS = 1e-6


def make_mitotar_config(d: dict | str, compute_dtype=torch.bfloat16) -> SimpleNamespace:
    """config.json (a dict or a path) -> the namespace the skeleton and the operators read."""
    if isinstance(d, str):
        with open(os.path.join(d, "config.json") if os.path.isdir(d) else d, encoding="utf-8") as f:
            d = json.load(f)
    if d.get("architecture") != "Mitotar":
        raise ValueError(f"not a Mitotar config: architecture = {d.get('architecture')!r}")
    layers = []
    for i, L in enumerate(d["layers"]):
        if L.get("type") != "parallel":
            raise ValueError(f"layer {i}: unknown layer type {L.get('type')!r}")
        left, right, mlp = L["mixer"]["left"], L["mixer"]["right"], L.get("mlp")
        if left["vdim"] != left["dim"]:
            raise ValueError(f"layer {i}: the left mixer's values are its keys, so vdim ({left['vdim']}) must equal dim ({left['dim']})")
        if left["heads"] % left["kv_heads"]:
            raise ValueError(f"layer {i}: heads ({left['heads']}) must be a multiple of kv_heads ({left['kv_heads']})")
        if mlp is not None and mlp.get("kind") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append(L)
    return SimpleNamespace(architectures=["Mitotar"], width=int(d["width"]), vocab=int(d["vocab"]), eps=float(d["norm"]["eps"]),
                           layers=layers, num_hidden_layers=len(layers), vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
                           compute_dtype=compute_dtype, max_position_embeddings=None, raw=d)


def mitotar_layer_specs(config) -> list:
    """What KHybridCache needs per layer: the key cache's (kv_heads, dim) and the recurrent state's (heads, dim, vdim)."""
    return [{"attn": (L["mixer"]["left"]["kv_heads"], L["mixer"]["left"]["dim"]),
             "rec": (L["mixer"]["right"]["heads"], L["mixer"]["right"]["dim"], L["mixer"]["right"]["vdim"])} for L in config.layers]


class MitotarEmbedding(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.vocab, self.width = config.vocab, config.width


class MitotarNorm(_Leaf):
    """unit RMS * (1 + w): the weight is stored around zero."""

    def __init__(self, width, eps, one_plus=True):
        super().__init__()
        self.width, self.eps, self.one_plus = width, eps, one_plus


class MitotarSigmoidAttention(_Leaf):
    def __init__(self, config, layer_idx, c):
        super().__init__()
        self.layer_idx, self.width, self.eps = layer_idx, config.width, config.eps
        self.heads, self.kv_heads, self.dim = int(c["heads"]), int(c["kv_heads"]), int(c["dim"])
        self.scale = float(c["scale"])
        self.temp_coef, self.temp_every = float(c["q_temp"]["coef"]), int(c["q_temp"]["every"])
        self.slope_span = DISTANCE_SLOPE_SPAN


class MitotarMLSTM(_Leaf):
    def __init__(self, config, layer_idx, c):
        super().__init__()
        self.layer_idx, self.width, self.eps = layer_idx, config.width, config.eps
        self.heads, self.dim, self.vdim, self.gate_cap = int(c["heads"]), int(c["dim"]), int(c["vdim"]), float(c["gate_cap"])
        self.denom_eps = MLSTM_DENOM_EPS


class MitotarParallelMixer(_Leaf):
    def __init__(self, config, layer_idx, c):
        super().__init__()
        self.eps = config.eps
        self.left = MitotarSigmoidAttention(config, layer_idx, c["left"])
        self.right = MitotarMLSTM(config, layer_idx, c["right"])


class MitotarMLP(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.ff = config.width, int(c["ff"])


class MitotarLayer(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        L = config.layers[layer_idx]
        self.mix = MitotarParallelMixer(config, layer_idx, L["mixer"])
        self.norm1 = MitotarNorm(config.width, config.eps)
        self.mlp = MitotarMLP(config, L["mlp"]) if L.get("mlp") is not None else None
        if self.mlp is not None:
            self.norm2 = MitotarNorm(config.width, config.eps)

    def forward(self, x, batch, cache):
        """x <- x + norm1(mix(x)); x <- x + norm2(mlp(x)): both sublayers read x itself, the norm sits on their output.  x is the fp32
        residual and is updated in place.  Operators that expose the fusion hooks take the norm and the residual and add in their last
        launch; otherwise the plain sequence."""
        if getattr(type(self.mix), "SUPPORTS_FUSION", False):
            self.mix(x, batch, cache, post_norm=self.norm1, residual=x)
        else:
            self.norm1(self.mix(x, batch, cache), residual=x)
        if self.mlp is not None:
            if getattr(type(self.mlp), "SUPPORTS_FUSION", False):
                self.mlp(x, post_norm=self.norm2, residual=x)
            else:
                self.norm2(self.mlp(x), residual=x)
        return x


class _Final(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.norm = MitotarNorm(config.width, config.eps)


class MitotarHead(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.in_features, self.out_features = config.width, config.vocab


class MitotarForCausalLM(nn.Module):
    """forward(input_ids, position_ids, past_key_values, cache_position, batch=, logits_rows=, last_token_only=) -> fp32 logits.

    With `batch` (a ForwardBatch planned by the KHybridCache in `past_key_values`): input_ids is the flattened token list of the
    step and the result is [len(logits_rows) or T, vocab].  Without it, the call is the single-sequence form the generation loop
    uses (util/generate.py): input_ids [1, T] at position_ids [1, T]; the result is [1, T or 1, vocab]."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed = MitotarEmbedding(config)
        for i in range(config.num_hidden_layers):
            self.add_module(f"l{i}", MitotarLayer(config, i))
        self.final = _Final(config)
        self.head = MitotarHead(config)

    def layers(self):
        return [getattr(self, f"l{i}") for i in range(self.config.num_hidden_layers)]

    def forward(self, input_ids=None, position_ids=None, past_key_values=None, cache_position=None, batch=None, logits_rows=None,
                last_token_only: bool = False, return_layers: bool = False):
        cache = past_key_values
        single = batch is None
        if single:
            batch = cache.single_request_batch(position_ids)
            if last_token_only and batch.T > 1:
                logits_rows = torch.tensor([batch.T - 1], dtype=torch.int32, device=cache.device)
        x = self.embed(input_ids, batch.positions)
        trail = []
        for layer in self.layers():
            x = layer(x, batch, cache)
            if return_layers:
                trail.append(x.clone())
        h = self.final.norm(x, rows=logits_rows, out_dtype=self.config.compute_dtype)
        logits = self.head(h)
        if single:
            logits = logits.unsqueeze(0)
        return (logits, torch.stack(trail)) if return_layers else logits
