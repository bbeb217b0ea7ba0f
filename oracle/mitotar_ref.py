"""TEST INFRASTRUCTURE ONLY — plain, slow torch statement of the Mitotar design, one function per mechanism, evaluated on the
CPU in fp64 (or fp32).  It shares no code with ktransformers_amd: the product's operators, cache and kernels are compared
with it.  Whole sequences only: no cache, no batching, no chunking — a sequence is a list of token ids.

Notation: x[t] is the residual stream at position t (positions count from 0), W a weight stored [out, in] and applied as
W @ h, `P[name]` a tensor of the checkpoint, `cfg` the parsed config.json."""
from __future__ import annotations

import math

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """The layer norm of the design: unit RMS times (1 + w), w stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sinusoid(positions: torch.Tensor, width: int) -> torch.Tensor:
    """[T, width]: entry 2i = sin(p * 10000^(-2i / width)), entry 2i + 1 = cos of the same angle."""
    out = torch.zeros(positions.numel(), width, dtype=torch.float64)
    p = positions.to(torch.float64)
    for e in range(width):
        i = e // 2
        ang = p * (10000.0 ** (-2.0 * i / width))
        out[:, e] = torch.sin(ang) if e % 2 == 0 else torch.cos(ang)
    return out


def embed(P, tokens: torch.Tensor, width: int, first_position: int = 0) -> torch.Tensor:
    pos = torch.arange(first_position, first_position + tokens.numel())
    return P["embed"][tokens] + sinusoid(pos, width).to(P["embed"].dtype)


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.div(positions + 1, every, rounding_mode="floor").to(torch.float64) + 1.0)


def distance_slopes(heads: int) -> torch.Tensor:
    """slope_h = 2^(-8 (h + 1) / heads)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=torch.float64)


def sigmoid_talk_attention(P, pre: str, c: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """The left mixer: grouped-query attention whose values are the un-normed keys, normed queries and keys, a query
    temperature that grows with the position, a linear distance bias, sigmoid weights (no softmax, no normalisation over
    keys) and a head-mixing matrix applied to the weights."""
    T = h.shape[0]
    H, G, D = c["heads"], c["kv_heads"], c["dim"]
    q = (h @ P[pre + ".q"].T).view(T, H, D)
    k = (h @ P[pre + ".k"].T).view(T, G, D)
    v = k                                                      # as projected, before the norm
    qn = norm_plain(q, P[pre + ".q.norm"], eps)
    kn = norm_plain(k, P[pre + ".k.norm"], eps)
    pos = torch.arange(T)
    qn = qn * query_temperature(pos, c["q_temp"]["coef"], c["q_temp"]["every"]).to(h.dtype).view(T, 1, 1)
    slopes = distance_slopes(H).to(h.dtype)
    rep = H // G
    w = torch.zeros(H, T, T, dtype=h.dtype)
    for hh in range(H):
        s = (qn[:, hh] @ kn[:, hh // rep].T) * c["scale"]
        dist = (pos.view(T, 1) - pos.view(1, T)).to(h.dtype)
        s = s - slopes[hh] * dist
        a = torch.sigmoid(s + P[pre + ".pb"][hh])
        w[hh] = torch.where(pos.view(T, 1) >= pos.view(1, T), a, torch.zeros_like(a))
    mixed = torch.einsum("hg,gij->hij", P[pre + ".talk"], w)
    out = torch.stack([mixed[hh] @ v[:, hh // rep] for hh in range(H)], dim=1)          # [T, H, D]
    return out.reshape(T, H * D) @ P[pre + ".o"].T


def mlstm_gates(P, pre: str, c: dict, h: torch.Tensor):
    """(log input gate, log forget gate), each [T, heads], soft-capped."""
    cap = c["gate_cap"]
    i = cap * torch.tanh((h @ P[pre + ".i"].T + P[pre + ".i.b"]) / cap)
    f = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ P[pre + ".f"].T + P[pre + ".f.b"]) / cap))
    return i, f


def mlstm_recurrence(q, k, v, i, f, state=None):
    """Token by token.  q, k [T, N, D], v [T, N, V], gates [T, N].  state = (S [N, D, V], n [N, D], m [N]) or None for
    the zero start (m starts at 0).  Returns o [T, N, V] and the final state."""
    T, N, D = q.shape
    V = v.shape[-1]
    if state is None:
        S = torch.zeros(N, D, V, dtype=q.dtype)
        n = torch.zeros(N, D, dtype=q.dtype)
        m = torch.zeros(N, dtype=q.dtype)
    else:
        S, n, m = (t.clone() for t in state)
    o = torch.zeros(T, N, V, dtype=q.dtype)
    for t in range(T):
        m_new = torch.maximum(f[t] + m, i[t])
        a = torch.exp(f[t] + m - m_new)
        b = torch.exp(i[t] - m_new)
        S = a.view(N, 1, 1) * S + b.view(N, 1, 1) * (k[t].unsqueeze(-1) * v[t].unsqueeze(-2))
        n = a.view(N, 1) * n + b.view(N, 1) * k[t]
        m = m_new
        num = torch.einsum("ndv,nd->nv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        o[t] = num / den.view(N, 1)
    return o, (S, n, m)


def mlstm_mixer(P, pre: str, c: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """The right mixer: matrix-memory recurrence, per-head unit norm, weight, output gate, projection."""
    T = h.shape[0]
    N, D, V = c["heads"], c["dim"], c["vdim"]
    q = (h @ P[pre + ".q"].T).view(T, N, D) * D ** -0.5
    k = (h @ P[pre + ".k"].T).view(T, N, D)
    v = (h @ P[pre + ".v"].T).view(T, N, V)
    i, f = mlstm_gates(P, pre, c, h)
    o, _ = mlstm_recurrence(q, k, v, i, f)
    o = unit_rms(o, eps).reshape(T, N * V) * P[pre + ".norm"]
    o = o * torch.sigmoid(h @ P[pre + ".g"].T)
    return o @ P[pre + ".o"].T


def parallel_mixer(P, pre: str, c: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """Both mixers read h; half the sum of their outputs, each normed over the width with its plain weight."""
    left = sigmoid_talk_attention(P, pre + ".left", c["left"], h, eps)
    right = mlstm_mixer(P, pre + ".right", c["right"], h, eps)
    return 0.5 * (norm_plain(left, P[pre + ".left.out"], eps) + norm_plain(right, P[pre + ".right.out"], eps))


def dense_mlp(P, pre: str, h: torch.Tensor) -> torch.Tensor:
    return gelu_tanh(h @ P[pre + ".up"].T) @ P[pre + ".down"].T


def forward(P, cfg: dict, tokens, dtype=torch.float64, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    P = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in P.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x = embed(P, tokens, cfg["width"])
    layers = []
    for li, layer in enumerate(cfg["layers"]):
        pre = f"l{li}"
        if layer["type"] != "parallel":
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + norm_one_plus(parallel_mixer(P, pre + ".mix", layer["mixer"], x, eps), P[pre + ".norm1"], eps)
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
            x = x + norm_one_plus(dense_mlp(P, pre + ".mlp", x), P[pre + ".norm2"], eps)
        layers.append(x.clone())
    logits = norm_one_plus(x, P["final.norm"], eps) @ P["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits


def random_checkpoint(cfg: dict, seed: int = 0, scale: float = 1.0) -> dict:
    """Random bf16-representable weights with the checkpoint's tensor names for a config of the design."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else scale / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    P = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W), "final.norm": vec(W)}
    for li, layer in enumerate(cfg["layers"]):
        p = f"l{li}"
        L, R = layer["mixer"]["left"], layer["mixer"]["right"]
        P[p + ".norm1"] = vec(W)
        P[p + ".mix.left.q"] = mat(L["heads"] * L["dim"], W)
        P[p + ".mix.left.k"] = mat(L["kv_heads"] * L["dim"], W)
        P[p + ".mix.left.q.norm"] = vec(L["dim"], 1.0)
        P[p + ".mix.left.k.norm"] = vec(L["dim"], 1.0)
        P[p + ".mix.left.talk"] = (torch.eye(L["heads"]) + 0.3 * torch.randn(L["heads"], L["heads"], generator=g)).to(torch.bfloat16)
        P[p + ".mix.left.pb"] = vec(L["heads"], -1.0, 0.5)
        P[p + ".mix.left.o"] = mat(W, L["heads"] * L["vdim"])
        P[p + ".mix.left.out"] = vec(W, 1.0)
        P[p + ".mix.right.q"] = mat(R["heads"] * R["dim"], W)
        P[p + ".mix.right.k"] = mat(R["heads"] * R["dim"], W)
        P[p + ".mix.right.v"] = mat(R["heads"] * R["vdim"], W)
        P[p + ".mix.right.g"] = mat(R["heads"] * R["vdim"], W)
        P[p + ".mix.right.o"] = mat(W, R["heads"] * R["vdim"])
        P[p + ".mix.right.norm"] = vec(R["heads"] * R["vdim"], 1.0)
        P[p + ".mix.right.i"] = mat(R["heads"], W)
        P[p + ".mix.right.i.b"] = vec(R["heads"], 0.0, 1.0)
        P[p + ".mix.right.f"] = mat(R["heads"], W)
        P[p + ".mix.right.f.b"] = vec(R["heads"], 3.0, 1.0)
        P[p + ".mix.right.out"] = vec(W, 1.0)
        if layer.get("mlp") is not None:
            P[p + ".norm2"] = vec(W)
            P[p + ".mlp.up"] = mat(layer["mlp"]["ff"], W)
            P[p + ".mlp.down"] = mat(W, layer["mlp"]["ff"])
    return P


def make_config(width=64, vocab=97, n_layers=2, heads=4, kv_heads=2, dim=16, r_heads=2, r_dim=8, r_vdim=16, ff=48, eps=1e-5,
                coef=0.25, every=8, scale=None, gate_cap=10.0, mlp_none_at=()) -> dict:
    """A small config of the design (the same keys config.json carries)."""
    layers = []
    for li in range(n_layers):
        layers.append({"type": "parallel",
                       "mixer": {"left": {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": dim,
                                          "q_temp": {"coef": coef, "every": every}, "scale": scale if scale is not None else dim ** -0.5},
                                 "right": {"dim": r_dim, "heads": r_heads, "vdim": r_vdim, "gate_cap": gate_cap}},
                       "mlp": None if li in mlp_none_at else {"ff": ff, "kind": "dense"}})
    return {"architecture": "Mitotar", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
