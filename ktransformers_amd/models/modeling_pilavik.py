"""Module skeleton of Pilavik — a pre- and post-normed decoder with an fp32 residual stream whose layers mix tokens either with a
gated delta rule (short convolutions in front, a matrix memory per head) or with a sliding-window latent attention with a softmax
sink, under a sigmoid-gated residual, with a PolyNorm feed-forward or a sigmoid-routed mixture of GLU experts, and a block of layers
that may run several times with the same weights.

Like the other skeletons of this package it only holds the structure the optimize rules inject into (optimize_rules/Pilavik.yaml)
and the glue (the order of layer runs, the layer's residual arrangement); every module that does arithmetic is a leaf that raises
until an operator replaces it.  Module paths equal the checkpoint's tensor prefixes:

    embed | loop | l<i>.{norm1,norm1b,norm2,norm2b} | l<i>.mix | l<i>.rg1 | l<i>.rg2 | l<i>.mlp | final.norm | head

config.json: {"architecture": "Pilavik", "width", "vocab", "norm": {"eps"}, "loop": {"start", "stop", "times"} | null,
"layers": [{"type": "delta", "mixer": {"heads", "kv_heads", "dim", "vdim", "conv"}, "mlp": ...} |
           {"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "mask": {"size"},
            "rot": {"base", "dims"}}, "mlp": ...}],
 mlp: null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "scale"}, "shared": {"ff"} | null}}.
Sizes and the constants listed there come from the file; what the design fixes is a constant here."""
from __future__ import annotations

import json
import os
from types import SimpleNamespace

import torch
from torch import nn

from ktransformers_amd.models.modeling_deepseek import _Leaf

# fixed by the design
DELTA_UNIT_EPS = 1e-6          # q, k -> x / sqrt(sum(x^2) + 1e-6)
ROUTER_SUM_EPS = 1e-20         # chosen scores / (their sum + 1e-20)
MIXER_TYPES = ("delta", "latent_attention")
MLP_KINDS = ("dense", "moe")


def make_pilavik_config(d: dict | str, compute_dtype=torch.bfloat16) -> SimpleNamespace:
    """config.json (a dict or a path) -> the namespace the skeleton and the operators read."""
    if isinstance(d, str):
        with open(os.path.join(d, "config.json") if os.path.isdir(d) else d, encoding="utf-8") as f:
            d = json.load(f)
    if d.get("architecture") != "Pilavik":
        raise ValueError(f"not a Pilavik config: architecture = {d.get('architecture')!r}")
    layers = list(d["layers"])
    for i, L in enumerate(layers):
        if L.get("type") not in MIXER_TYPES:
            raise ValueError(f"layer {i}: unknown layer type {L.get('type')!r}")
        m = L["mixer"]
        if L["type"] == "delta" and m["heads"] % m["kv_heads"]:
            raise ValueError(f"layer {i}: heads ({m['heads']}) must be a multiple of kv_heads ({m['kv_heads']})")
        if L["type"] == "latent_attention":
            rot = m.get("rot") or {"dims": 0, "base": 1.0}
            if rot["dims"] % 2 or rot["dims"] > m["rot_dim"]:
                raise ValueError(f"layer {i}: rot.dims ({rot['dims']}) must be even and at most rot_dim ({m['rot_dim']})")
        if L.get("mlp") is not None and L["mlp"].get("kind") not in MLP_KINDS:
            raise ValueError(f"layer {i}: unknown feed-forward kind {L['mlp'].get('kind')!r}")
    loop = d.get("loop") or None
    if loop is not None:
        loop = {"start": int(loop["start"]), "stop": int(loop["stop"]), "times": int(loop["times"])}
        if not (0 <= loop["start"] < loop["stop"] <= len(layers)) or loop["times"] < 1:
            raise ValueError(f"loop {loop} does not fit {len(layers)} layers")
    runs = layer_runs(len(layers), loop)
    return SimpleNamespace(architectures=["Pilavik"], width=int(d["width"]), vocab=int(d["vocab"]), eps=float(d["norm"]["eps"]),
                           layers=layers, loop=loop, runs=runs, num_hidden_layers=len(layers), vocab_size=int(d["vocab"]),
                           hidden_size=int(d["width"]), compute_dtype=compute_dtype, max_position_embeddings=None, raw=d)


def layer_runs(n_layers: int, loop: dict | None) -> list:
    """The order in which layers run: [(layer index, pass number when this run opens a pass of the repeated block, else None)]."""
    if not loop:
        return [(i, None) for i in range(n_layers)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n_layers)]


def pilavik_layer_specs(config) -> list:
    """What KHybridCache needs, one entry per layer RUN (each pass of the repeated block has its own cache or state)."""
    specs = []
    for i, _ in config.runs:
        L = config.layers[i]
        m = L["mixer"]
        if L["type"] == "delta":
            channels = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
            specs.append({"delta": (m["heads"], m["dim"], m["vdim"]), "conv": (channels, int(m.get("conv", 1)))})
        else:
            specs.append({"latent": m["kv_rank"] + m["rot_dim"]})
    return specs


class PilavikEmbedding(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.vocab, self.width = config.vocab, config.width


class PilavikNorm(_Leaf):
    def __init__(self, width, eps):
        super().__init__()
        self.width, self.eps = width, eps


class PilavikPassOffset(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.width, self.times = config.width, config.loop["times"]


class PilavikGate(_Leaf):
    """The residual gate's linear: sigmoid(W h + b) multiplies a sublayer's result."""

    def __init__(self, width):
        super().__init__()
        self.in_features = self.out_features = width


class PilavikDeltaMixer(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps, self.unit_eps = config.width, config.eps, DELTA_UNIT_EPS
        self.heads, self.kv_heads, self.dim, self.vdim = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        self.taps = int(c.get("conv", 1))


class PilavikLatentAttention(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps = config.width, config.eps
        self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = (int(c[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale = float(c["scale"])
        self.window = int((c.get("mask") or {}).get("size") or 0)
        rot = c.get("rot") or {"dims": 0, "base": 1.0}
        self.rot_dims, self.rot_base = int(rot["dims"]), float(rot["base"])


class PilavikDenseMLP(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width, self.eps, self.ff = config.width, config.eps, int(c["ff"])


class PilavikMoE(_Leaf):
    def __init__(self, config, c):
        super().__init__()
        self.width = config.width
        self.experts, self.top, self.route_scale = int(c["router"]["experts"]), int(c["router"]["top"]), float(c["router"].get("scale", 1.0))
        self.sum_eps = ROUTER_SUM_EPS
        self.ff = int(c["expert"]["ff"])
        self.shared_ff = int(c["shared"]["ff"]) if c.get("shared") else 0


class PilavikLayer(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        L = config.layers[layer_idx]
        W, eps = config.width, config.eps
        self.norm1, self.norm1b, self.rg1 = PilavikNorm(W, eps), PilavikNorm(W, eps), PilavikGate(W)
        self.mix = PilavikDeltaMixer(config, L["mixer"]) if L["type"] == "delta" else PilavikLatentAttention(config, L["mixer"])
        c = L.get("mlp")
        self.mlp = None if c is None else (PilavikDenseMLP(config, c) if c["kind"] == "dense" else PilavikMoE(config, c))
        if self.mlp is not None:
            self.norm2, self.norm2b, self.rg2 = PilavikNorm(W, eps), PilavikNorm(W, eps), PilavikGate(W)

    def forward(self, x, batch, cache, cache_idx, h=None, next_norm=None):
        """x <- x + norm1b(mix(h) * sigmoid(rg1 h)), h = norm1(x); then the same with the feed-forward.  x is the fp32 residual and is
        updated in place.  The gate's product rides in the sublayer's input GEMM; gate, post-norm, output bias, the mixture's weighted
        sum, the residual add AND the pre-norm of whatever follows are the post-norm's one launch: `h` is norm1(x) when the caller
        already has it, `next_norm` the pre-norm of the next layer run; returns (x, next_norm(x) or None)."""
        fused = hasattr(self.norm1b, "gated_add") and hasattr(self.norm1, "weight_f32")

        def after(post, nxt, **kw):
            if nxt is not None and fused:
                return post.gated_add(x, next_norm=nxt, **kw)[1]
            post.gated_add(x, **kw)
            return nxt(x) if nxt is not None else None

        if h is None:
            h = self.norm1(x)
        y, gl = self.mix(h, batch, cache, cache_idx, rider=self.rg1)
        h = after(self.norm1b, self.norm2 if self.mlp is not None else next_norm, y=y, gate_logits=gl, gate_bias=self.rg1.bias_f32)
        if self.mlp is not None:
            if getattr(self.mlp, "RETURNS_EXPERT_ROWS", False):
                y, gl, rows, pair_pos, topk_w = self.mlp(h, rider=self.rg2)
                h = after(self.norm2b, next_norm, y=y, gate_logits=gl, gate_bias=self.rg2.bias_f32, expert_rows=rows, pair_pos=pair_pos,
                          topk_w=topk_w)
            else:
                y, gl = self.mlp(h, rider=self.rg2)
                h = after(self.norm2b, next_norm, y=y, ybias=self.mlp.down_bias, gate_logits=gl, gate_bias=self.rg2.bias_f32)
        return x, h


class _Final(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.norm = PilavikNorm(config.width, config.eps)


class PilavikHead(_Leaf):
    def __init__(self, config):
        super().__init__()
        self.in_features, self.out_features = config.width, config.vocab


class PilavikForCausalLM(nn.Module):
    """forward(input_ids, position_ids, past_key_values, cache_position, batch=, logits_rows=, last_token_only=) -> fp32 logits.

    With `batch` (a ForwardBatch planned by the KHybridCache in `past_key_values`): input_ids is the flattened token list of the
    step and the result is [len(logits_rows) or T, vocab].  Without it, the call is the single-sequence form the generation loop
    uses (util/generate.py): input_ids [1, T] at position_ids [1, T]; the result is [1, T or 1, vocab]."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed = PilavikEmbedding(config)
        if config.loop is not None:
            self.loop = PilavikPassOffset(config)
        for i in range(config.num_hidden_layers):
            self.add_module(f"l{i}", PilavikLayer(config, i))
        self.final = _Final(config)
        self.head = PilavikHead(config)

    def forward(self, input_ids=None, position_ids=None, past_key_values=None, cache_position=None, batch=None, logits_rows=None,
                last_token_only: bool = False, return_layers: bool = False):
        cache = past_key_values
        single = batch is None
        if single:
            batch = cache.single_request_batch(position_ids)
            if last_token_only and batch.T > 1:
                logits_rows = torch.tensor([batch.T - 1], dtype=torch.int32, device=cache.device)
        x = self.embed(input_ids, batch.positions)
        x0 = x.clone() if self.config.loop is not None and self.config.loop["times"] > 1 else None
        trail, h, runs = [], None, self.config.runs
        for run, (i, opens_pass) in enumerate(runs):
            if opens_pass is not None:
                self.loop(x, x0, opens_pass)
            # the pre-norm of the next run is computed by this run's last launch, unless something is added to x in between
            follows = getattr(self, f"l{runs[run + 1][0]}").norm1 if run + 1 < len(runs) and runs[run + 1][1] is None else None
            x, h = getattr(self, f"l{i}")(x, batch, cache, run, h=h, next_norm=follows)
            if return_layers:
                trail.append(x.clone())
        h = self.final.norm(x, rows=logits_rows, out_dtype=self.config.compute_dtype)
        logits = self.head(h)
        if single:
            logits = logits.unsqueeze(0)
        return (logits, torch.stack(trail)) if return_layers else logits
