"""TEST INFRASTRUCTURE ONLY — plain, slow torch statement of the Pilavik design, one function per mechanism, evaluated on the
CPU in fp64 (or fp32).  It shares no code with ktransformers_amd: the product's operators, cache and kernels are compared
with it.  Whole sequences only: no cache, no batching, no chunking — a sequence is a list of token ids.

Notation: x[t] is the residual stream at position t (positions count from 0), W a weight stored [out, in] and applied as
W @ h, `P[name]` a tensor of the checkpoint, `cfg` the parsed config.json."""
from __future__ import annotations

import math

import torch

UNIT_EPS = 1e-6        # inside the root of the delta mixer's unit vectors
ROUTER_SUM_EPS = 1e-20


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt(d.pow(2).mean(dim=-1, keepdim=True) + eps) * w + b


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def short_conv(x, taps):
    """x [T, C], taps [C, K] (last column multiplies the current token): y[t, c] = sum_j taps[c, K-1-j] x[t-j, c], zeros before 0."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        if j < T:
            y[j:] += x[:T - j] * taps[:, K - 1 - j]
    return y


def delta_mixer(P, pre, c, h, eps):
    """Gated delta rule: per head a [dim, vdim] memory S; S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(short_conv(h @ P[pre + "q"].T, P[pre + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ P[pre + "k"].T, P[pre + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ P[pre + "v"].T, P[pre + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + UNIT_EPS) * D ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + UNIT_EPS)
    beta = torch.sigmoid(h @ P[pre + "b"].T)                                                   # [T, H]
    g = torch.exp(-torch.exp(P[pre + "A_log"]) * softplus(h @ P[pre + "a"].T + P[pre + "dt_bias"]))   # [T, H]
    gate = silu(h @ P[pre + "g"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    rep = H // G
    for hd in range(H):
        S = torch.zeros(D, V, dtype=h.dtype)
        kh = hd // rep
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hd] = S.T @ q[t, kh]
    o = unit_rms(o, eps) * P[pre + "norm"] * gate
    return o.reshape(T, H * V) @ P[pre + "o"].T


def rotate_pairs(x, positions, base, dims):
    """Interleaved rotary: the first `dims` entries of the last axis, pair (2i, 2i+1), angle p * base^(-2i/dims).  x [T, ..., n]."""
    out = x.clone()
    p = positions.to(x.dtype)
    for i in range(dims // 2):
        a = p * (base ** (-2.0 * i / dims))
        cs, sn = torch.cos(a), torch.sin(a)
        while cs.dim() < x.dim() - 1:
            cs, sn = cs.unsqueeze(-1), sn.unsqueeze(-1)
        u, w = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * cs - w * sn
        out[..., 2 * i + 1] = w * cs + u * sn
    return out


def latent_attention(P, pre, c, h, eps):
    """Keys and values expanded from a normed latent; one rotated key part shared by the heads; sliding window; sink in the softmax."""
    T = h.shape[0]
    H, D, R, V, L = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    pos = torch.arange(T)
    q = (h @ P[pre + "q"].T).view(T, H, D + R)
    rot = c.get("rot") or {"base": 1.0, "dims": 0}
    qn, qr = q[..., :D], rotate_pairs(q[..., D:], pos, rot["base"], rot["dims"])
    dkv = h @ P[pre + "dkv"].T
    lat = unit_rms(dkv[:, :L], eps) * P[pre + "dkv.norm"]
    kr = rotate_pairs(dkv[:, L:], pos, rot["base"], rot["dims"])                              # [T, R]
    kn = (lat @ P[pre + "uk"].T).view(T, H, D)
    val = (lat @ P[pre + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    W = (c.get("mask") or {}).get("size") or T + 1          # no mask: every earlier position is seen
    for i in range(T):
        lo = max(0, i - W + 1)
        for hd in range(H):
            s = (kn[lo:i + 1, hd] @ qn[i, hd] + kr[lo:i + 1] @ qr[i, hd]) * c["scale"]
            sink = P[pre + "sink"][hd]
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            out[i, hd] = (e / (e.sum() + torch.exp(sink - m))) @ val[lo:i + 1, hd]
    return out.reshape(T, H * V) @ P[pre + "o"].T


def poly_norm(z, coef, eps):
    a, b, c, e = coef
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(P, pre, h, eps):
    z = h @ P[pre + "up"].T + P[pre + "up.b"]
    return poly_norm(z, P[pre + "act"], eps) @ P[pre + "down"].T + P[pre + "down.b"]


def glu_expert(P, pre, h):
    return (silu(h @ P[pre + "gate"].T) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def moe_ff(P, pre, c, h):
    T = h.shape[0]
    s = torch.sigmoid(h @ P[pre + "router"].T)
    top = c["router"]["top"]
    out = torch.zeros(T, P[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(T):
        idx = torch.topk(s[t], top).indices
        w = s[t, idx] / (s[t, idx].sum() + ROUTER_SUM_EPS) * c["router"]["scale"]
        for j, e in enumerate(idx.tolist()):
            out[t] += w[j] * glu_expert(P, f"{pre}e{e}.", h[t:t + 1])[0]
    if c.get("shared") is not None:
        out = out + glu_expert(P, pre + "shared.", h)
    return out


def layer(P, cfg, i, x):
    L, pre, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    ln = lambda name, z: layer_norm(z, P[pre + name], P[pre + name + ".b"], eps)
    h = ln("norm1", x)
    y = {"delta": delta_mixer, "latent_attention": latent_attention}[L["type"]](P, pre + "mix.", L["mixer"], h, eps)
    y = y * torch.sigmoid(h @ P[pre + "rg1"].T + P[pre + "rg1.b"])
    x = x + ln("norm1b", y)
    if L.get("mlp") is not None:
        h = ln("norm2", x)
        y = dense_ff(P, pre + "mlp.", h, eps) if L["mlp"]["kind"] == "dense" else moe_ff(P, pre + "mlp.", L["mlp"], h)
        y = y * torch.sigmoid(h @ P[pre + "rg2"].T + P[pre + "rg2.b"])
        x = x + ln("norm2b", y)
    return x


def layer_runs(cfg):
    """The order in which layers run: layers start .. stop-1 repeated `times` times in place.  -> [(layer index, pass number or None)]."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None, False) for i in range(loop["stop"], n)]


def forward(P, cfg, tokens, return_layers=False):
    """tokens: a list of ids or a 1-D LongTensor -> logits [T, vocab] (and the residual stream after every layer run)."""
    x0 = P["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x, trail = x0.clone(), []
    for i, t, first in layer_runs(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + P["loop.step"][t]
        x = layer(P, cfg, i, x)
        trail.append(x)
    eps = cfg["norm"]["eps"]
    logits = layer_norm(x, P["final.norm"], P["final.norm.b"], eps) @ P["head"].T
    return (logits, torch.stack(trail)) if return_layers else logits


# ---- small random models for the tests ------------------------------------------------------------------------------------------
def delta_layer(heads=4, kv_heads=2, dim=16, vdim=16, conv=3, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def attention_layer(heads=3, dim=16, rot_dim=8, vdim=16, kv_rank=24, window=12, rot_dims=None, base=10000.0, scale=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
         "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense_mlp(ff=48):
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=6, top=2, ff=24, scale=1.25, shared_ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale},
            "shared": {"ff": shared_ff} if shared_ff else None}


def make_config(layers, width=32, vocab=61, eps=1e-5, loop=None):
    return {"architecture": "Pilavik", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers, "loop": loop}


def random_checkpoint(cfg: dict, seed: int = 0) -> dict:
    """Random bf16-representable weights with the checkpoint's tensor names for a config of the design."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + torch.randn(n, generator=g) * s).to(torch.bfloat16)

    P = {"embed": mat(cfg["vocab"], W, 1.0), "head": mat(cfg["vocab"], W), "final.norm": vec(W, 1.0), "final.norm.b": vec(W)}
    if cfg.get("loop"):
        P["loop.step"] = mat(cfg["loop"]["times"], W, 0.3)
    for li, layer in enumerate(cfg["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.get("mlp") else ()):
            P[p + n], P[p + n + ".b"] = vec(W, 1.0), vec(W)
        for n in ("rg1",) + (("rg2",) if layer.get("mlp") else ()):
            P[p + n], P[p + n + ".b"] = mat(W, W), vec(W, 0.5, 0.5)
        if layer["type"] == "delta":
            H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            P[p + "mix.q"], P[p + "mix.k"], P[p + "mix.v"] = mat(G * D, W, 1.0), mat(G * D, W, 1.0), mat(H * V, W, 1.0)
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                P[p + f"mix.{n}.conv"] = mat(rows, K, 0.6)
            P[p + "mix.b"], P[p + "mix.a"], P[p + "mix.g"] = mat(H, W), mat(H, W), mat(H * V, W)
            P[p + "mix.A_log"], P[p + "mix.dt_bias"] = vec(H, -1.0, 0.7), vec(H, -1.0, 1.0)
            P[p + "mix.norm"], P[p + "mix.o"] = vec(V, 1.0), mat(W, H * V)
        else:
            H, D, R, V, L = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            P[p + "mix.q"], P[p + "mix.dkv"] = mat(H * (D + R), W, 2.0 / math.sqrt(W)), mat(L + R, W, 2.0 / math.sqrt(W))
            P[p + "mix.dkv.norm"] = vec(L, 1.0)
            P[p + "mix.uk"], P[p + "mix.uv"] = mat(H * D, L), mat(H * V, L)
            P[p + "mix.sink"], P[p + "mix.o"] = vec(H, 0.0, 1.0), mat(W, H * V)
        c = layer.get("mlp")
        if c and c["kind"] == "dense":
            P[p + "mlp.up"], P[p + "mlp.up.b"] = mat(c["ff"], W), vec(c["ff"])
            P[p + "mlp.down"], P[p + "mlp.down.b"] = mat(W, c["ff"]), vec(W)
            P[p + "mlp.act"] = torch.tensor([0.6, 0.3, 0.2, 0.1]).to(torch.bfloat16) + vec(4, 0.0, 0.05)
        elif c:
            F = c["expert"]["ff"]
            P[p + "mlp.router"] = mat(c["router"]["experts"], W, 2.0 / math.sqrt(W))
            for e in range(c["router"]["experts"]):
                P[p + f"mlp.e{e}.gate"], P[p + f"mlp.e{e}.up"], P[p + f"mlp.e{e}.down"] = mat(F, W), mat(F, W), mat(W, F)
            if c.get("shared"):
                SF = c["shared"]["ff"]
                P[p + "mlp.shared.gate"], P[p + "mlp.shared.up"], P[p + "mlp.shared.down"] = mat(SF, W), mat(SF, W), mat(W, SF)
    return P


def as_double(P: dict) -> dict:
    return {k: v.double() for k, v in P.items()}
