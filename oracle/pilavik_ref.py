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
    qn, qr = q[..., :D], rotate_pairs(q[..., D:], pos, c["rot"]["base"], c["rot"]["dims"])
    dkv = h @ P[pre + "dkv"].T
    lat = unit_rms(dkv[:, :L], eps) * P[pre + "dkv.norm"]
    kr = rotate_pairs(dkv[:, L:], pos, c["rot"]["base"], c["rot"]["dims"])                    # [T, R]
    kn = (lat @ P[pre + "uk"].T).view(T, H, D)
    val = (lat @ P[pre + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    W = c["mask"]["size"]
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
    """tokens: 1-D LongTensor -> logits [T, vocab] (and the residual stream after every layer run)."""
    x0 = P["embed"][tokens]
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
