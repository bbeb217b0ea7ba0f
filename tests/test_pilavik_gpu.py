"""Pilavik on the GPU against the plain CPU statement of the design (oracle/pilavik_ref.py, fp64): every mechanism alone through its
kernels and operator, then the model through the framework's registry, cache manager, step function and generation loops — whole
prompts, token-by-token decoding, portions, unequal batches, reused pages and slots, keys at the window's edge and at page borders,
odd sizes.  Small random configurations; fp32 runs are held to rounding, bf16 runs to bf16 rounding."""
import math

import pytest
import torch

from oracle import pilavik_ref as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 3e-4, BF16: 6e-2}


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def rows_rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float(((got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)).max())


def rows_close(got, ref, dtype, f32_tol=None):
    """Logit rows against the plain statement.  fp32: every row to rounding.  bf16: rows to bf16 rounding — except that a router score
    within rounding of the next expert's may pick the other expert for a token, which moves that row (and, through the recurrent
    layers, some later ones) by more: the median row is held to the bf16 bound, at most one row in five may exceed twice that, none
    by a gross amount."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    e = (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt().clamp_min(1e-30)
    if dtype == F32:
        return float(e.max()) < (f32_tol or TOL[F32])
    return float(e.max()) < 0.5 and float(e.median()) < TOL[BF16] and int((e > 0.12).sum()) <= max(1, e.numel() // 5)


def build(cfg, seed, dtype, max_tokens=2048, max_requests=8, page_size=16, P=None):
    from ktransformers_amd.models import load_model
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_pilavik import pilavik_layer_specs
    from ktransformers_amd.util.loader import DictLoader
    P = R.random_checkpoint(cfg, seed) if P is None else P
    model, config, _ = load_model(cfg, dtype=dtype, device=DEV, loader=DictLoader(P))
    cache = KHybridCache(pilavik_layer_specs(config), max_tokens, max_requests=max_requests, page_size=page_size, dtype=dtype, device=DEV)
    return model, cache, R.as_double(P)


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def engine_of(model, cache, **kw):
    from ktransformers_amd.util.batch_engine import BatchEngine
    return BatchEngine(model, cache, **kw)


def steps(eng, rid, toks, sizes, end=True):
    """Feed toks in portions of the given sizes; logits of every position."""
    got, at = [], 0
    for n in sizes:
        last = at + n == len(toks)
        got.append(eng.step([{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}], [rid] if last and end else []))
        at += n
    assert at == len(toks)
    return torch.cat(got)


CONFIGS = {
    # delta / attention alternating, dense and mixture feed-forwards, a repeated block of two layers
    "loop": lambda: R.make_config([R.delta_layer(mlp=R.dense_mlp()), R.attention_layer(mlp=R.moe_mlp()), R.delta_layer(mlp=R.moe_mlp()),
                                   R.attention_layer(heads=2, window=7, mlp=R.dense_mlp())], loop={"start": 1, "stop": 3, "times": 3}),
    # nothing a multiple of anything: odd width and vocab, 3 heads over 1 key head, 2 taps, partial rotation, no shared expert, top = 1
    "odd": lambda: R.make_config([R.attention_layer(heads=5, dim=12, rot_dim=6, vdim=10, kv_rank=9, window=5, rot_dims=4, base=77.0,
                                                    mlp=R.moe_mlp(experts=3, top=1, ff=7, scale=0.8, shared_ff=0)),
                                  R.delta_layer(heads=3, kv_heads=1, dim=5, vdim=7, conv=2, mlp=None),
                                  R.delta_layer(heads=2, kv_heads=2, dim=12, vdim=80, conv=4, mlp=R.dense_mlp(ff=21))],
                                 width=40, vocab=53, eps=1e-3),
    # sizes the matrix-core paths take; the whole model is the repeated block; no window on one layer; every expert chosen
    "wide": lambda: R.make_config([R.attention_layer(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=64, window=None,
                                                     mlp=R.moe_mlp(experts=4, top=4, ff=32, shared_ff=64)),
                                   R.delta_layer(heads=4, kv_heads=4, dim=32, vdim=64, conv=3, mlp=R.dense_mlp(ff=128))],
                                  width=128, vocab=200, loop={"start": 0, "stop": 2, "times": 2}),
    # no repeated block, taps = 1, window = 1 (a token sees itself only), rotation switched off
    "plain": lambda: R.make_config([R.delta_layer(heads=1, kv_heads=1, dim=16, vdim=16, conv=1, mlp=R.moe_mlp(experts=8, top=3)),
                                    R.attention_layer(heads=1, window=1, rot_dims=0, mlp=None)], width=24, loop=None),
}


# ---- mechanisms alone ----------------------------------------------------------------------------------------------------------
def test_layer_norm_and_gated_post_norm():
    from ktransformers_amd._native_hyb import gated_norm_add, layer_norm, rows_add
    g = torch.Generator().manual_seed(3)
    d = lambda t: None if t is None else t.to(DEV)
    for W in (48, 37, 300, 5000):
        x, y, gl = (torch.randn(6, W, generator=g) * 3 + 1 for _ in range(3))
        w, b, yb, gb = (torch.randn(W, generator=g) for _ in range(4))
        eps = 1e-3
        for dt in (F32, BF16):
            assert rel(layer_norm(d(x), d(w), d(b), eps, out_dtype=dt), R.layer_norm(x.double(), w.double(), b.double(), eps)) < (1e-6 if dt == F32 else 4e-3)
        rows = torch.tensor([5, 0, 0, 2], dtype=torch.int32)
        assert rel(layer_norm(d(x), d(w), None, eps, rows=d(rows)), R.layer_norm(x.double(), w.double(), 0.0, eps)[rows.long()]) < 1e-6
        # gate, output bias, strided inputs (columns of a wider tensor)
        wide = torch.cat([torch.randn(6, 3, generator=g), y, gl], dim=1).to(DEV)
        xr = d(x.clone())
        gated_norm_add(xr, d(w), d(b), eps, y=wide[:, 3:3 + W], ybias=d(yb), gate_logits=wide[:, 3 + W:], gate_bias=d(gb))
        z = (y.double() + yb.double()) * torch.sigmoid(gl.double() + gb.double())
        assert rel(xr, x.double() + R.layer_norm(z, w.double(), b.double(), eps)) < 1e-6
        # the gathered, weighted expert rows
        top = 3
        er = torch.randn(6 * top, W, generator=g)
        pos = torch.randperm(6 * top, generator=g).int()
        tw = torch.rand(6, top, generator=g)
        xr = d(x.clone())
        gated_norm_add(xr, d(w), None, eps, y=d(y), gate_logits=d(gl), expert_rows=d(er), pair_pos=d(pos), topk_w=d(tw))
        mix = (er.double()[pos.long()].view(6, top, W) * tw.double().unsqueeze(-1)).sum(1)
        z = (y.double() + mix) * torch.sigmoid(gl.double())
        assert rel(xr, x.double() + R.layer_norm(z, w.double(), 0.0, eps)) < 1e-6
        xr = d(x.clone())
        gated_norm_add(xr, d(w), d(b), eps, expert_rows=d(er), pair_pos=d(pos), topk_w=d(tw))
        assert rel(xr, x.double() + R.layer_norm(mix, w.double(), b.double(), eps)) < 1e-6
        for dt in (F32, BF16):      # the pre-norm of what follows, from the same launch
            xr = d(x.clone())
            xr2, hn = gated_norm_add(xr, d(w), d(b), eps, y=d(y), ybias=d(yb), gate_logits=d(gl), gate_bias=d(gb), next_norm=(d(gb), d(yb), 2 * eps, dt))
            z = (y.double() + yb.double()) * torch.sigmoid(gl.double() + gb.double())
            xn = x.double() + R.layer_norm(z, w.double(), b.double(), eps)
            assert xr2 is xr and rel(xr, xn) < 1e-6 and rel(hn, R.layer_norm(xn, gb.double(), yb.double(), 2 * eps)) < (2e-6 if dt == F32 else 4e-3)
        xr = d(x.clone())
        rows_add(xr, d(y), d(w))
        assert rel(xr, x.double() + y.double() + w.double()) < 1e-7
        xr = d(x.clone())
        rows_add(xr, None, d(w))
        assert rel(xr, x.double() + w.double()) < 1e-7


@pytest.mark.parametrize("F", [16, 37, 700])
def test_poly_norm(F):
    from ktransformers_amd._native_hyb import poly_norm
    g = torch.Generator().manual_seed(F)
    z, bias, coef = torch.randn(5, F + 3, generator=g) * 2, torch.randn(F, generator=g), torch.tensor([0.7, -0.3, 0.2, 0.05])
    ref = R.poly_norm(z[:, 3:].double() + bias.double(), coef.double(), 1e-4)
    got = poly_norm(z.to(DEV)[:, 3:], bias.to(DEV), coef.to(DEV), 1e-4)
    assert rel(got, ref) < 1e-6
    assert rel(poly_norm(z.to(DEV)[:, 3:], bias.to(DEV), coef.to(DEV), 1e-4, out_dtype=BF16), ref) < 4e-3


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("G,M,N,K", [(1, 5, 7, 9), (3, 70, 24, 16), (5, 33, 130, 40), (2, 129, 64, 96)])
def test_per_head_products(dtype, G, M, N, K):
    from ktransformers_amd._native_hyb import head_gemm
    g = torch.Generator().manual_seed(G * 100 + M)
    a = torch.randn(M, 3 + G * (K + 2), generator=g).to(BF16).float()
    w = torch.randn(G, N, K, generator=g).to(BF16).float()
    out = torch.zeros(M, G * N + 1, dtype=torch.float32, device=DEV)
    head_gemm(a.to(dtype).to(DEV)[:, 3:], K + 2, w.to(dtype).to(DEV), out[:, 1:], N)
    for h in range(G):
        ref = a[:, 3 + h * (K + 2):3 + h * (K + 2) + K].double() @ w[h].double().T
        assert rel(out[:, 1 + h * N:1 + (h + 1) * N], ref) < 1e-6, h
    assert float(out[:, 0].abs().max()) == 0.0


@pytest.mark.parametrize("E,top,T", [(6, 2, 50), (3, 1, 7), (4, 4, 9), (70, 5, 300), (16, 2, 1)])
def test_router_and_expert_sort(E, top, T):
    from ktransformers_amd._native_hyb import moe_plan, moe_route
    g = torch.Generator().manual_seed(E * 10 + top)
    logits = torch.randn(T, E + 2, generator=g) * 2
    idx, w = moe_route(logits.to(DEV)[:, 1:1 + E], top, 1.7, 1e-20)
    s = torch.sigmoid(logits[:, 1:1 + E].double())
    ref = s.topk(top, dim=-1)
    assert torch.equal(idx.cpu().long().sort(-1).values, ref.indices.sort(-1).values)
    got_w = torch.zeros(T, E, dtype=torch.float64).scatter_(1, idx.cpu().long(), w.cpu().double())
    ref_w = torch.zeros(T, E, dtype=torch.float64).scatter_(1, ref.indices, ref.values / ref.values.sum(-1, keepdim=True) * 1.7)
    assert (got_w - ref_w).abs().max() < 1e-6
    plan = moe_plan(idx, E)
    off, st, pp = plan.group_off.cpu().tolist(), plan.sorted_tok.cpu().tolist(), plan.pair_pos.cpu().tolist()
    flat = idx.cpu().flatten().tolist()
    assert off[0] == 0 and off[-1] == T * top and sorted(pp) == list(range(T * top))
    for pair, e in enumerate(flat):
        assert off[e] <= pp[pair] < off[e + 1] and st[pp[pair]] == pair // top
    nt = int(plan.num_tiles.cpu())
    tiles = list(zip(plan.tile_group.cpu().tolist()[:nt], plan.tile_row0.cpu().tolist()[:nt]))
    want = [(e, r) for e in range(E) for r in range(off[e], off[e + 1], 64)]
    assert tiles == want and nt <= plan.max_tiles
    assert plan.sorted_group.cpu().tolist() == [e for e in range(E) for _ in range(off[e], off[e + 1])]
    wide = moe_plan(idx, E, wide=True)          # 128-row tiles (what prompt-sized bf16 steps take)
    off = wide.group_off.cpu().tolist()
    nt = int(wide.num_tiles.cpu())
    assert list(zip(wide.tile_group.cpu().tolist()[:nt], wide.tile_row0.cpu().tolist()[:nt])) == \
        [(e, r) for e in range(E) for r in range(off[e], off[e + 1], 128)] and nt <= wide.max_tiles


def _operator(cfg, seed, dtype, page_size=8, P=None):
    """A one-layer model without feed-forward whose mixer operator, cache and batch plans the tests drive directly."""
    model, cache, P = build(cfg, seed, dtype, page_size=page_size, P=P)
    return model.l0.mix, cache, P


def _mixer_in_portions(op, cache, h, dtype, sizes, rid="r"):
    cache.admit(rid)
    out, at = [], 0
    for n in sizes:
        fb = cache.plan([(rid, n)])
        y, rider = op(h[at:at + n].to(dtype).to(DEV), fb, cache, 0)
        assert rider is None
        out.append(y)
        at += n
    cache.release(rid)
    return torch.cat(out)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H,G,D,V,taps", [(4, 2, 16, 16, 3), (3, 1, 5, 7, 2), (2, 2, 40, 72, 4), (1, 1, 24, 80, 1), (2, 1, 130, 33, 3), (6, 3, 64, 64, 3)])
def test_delta_rule_whole_portions_and_state_carry(dtype, H, G, D, V, taps):
    cfg = R.make_config([R.delta_layer(heads=H, kv_heads=G, dim=D, vdim=V, conv=taps)], width=24)
    op, cache, P = _operator(cfg, 5, dtype)
    g = torch.Generator().manual_seed(7)
    T = 37
    h = torch.randn(T, 24, generator=g).to(BF16).float()
    ref = R.delta_mixer(P, "l0.mix.", cfg["layers"][0]["mixer"], h.double(), cfg["norm"]["eps"])
    tol = 2e-5 if dtype == F32 else 3e-2
    for t in cache.state_tensors():       # a fresh request must not see what its slot held
        t.fill_(7.0)
    for sizes in ([T], [1] * T, [2] * 18 + [1], [5, 1, 1, 13, 2, 15], [36, 1]):
        assert rel(_mixer_in_portions(op, cache, h, dtype, sizes), ref) < tol, sizes


def test_delta_rule_remembers_far_tokens():
    """Slow decay (A_log very negative): what the first tokens wrote is still read hundreds of tokens later, through prompts cut at
    any place and through decode steps."""
    cfg = R.make_config([R.delta_layer(heads=2, kv_heads=1, dim=16, vdim=16, conv=3)], width=24)
    P = R.random_checkpoint(cfg, 2)
    P["l0.mix.A_log"] = torch.full((2,), -9.0).to(BF16)
    op, cache, Pd = _operator(cfg, 2, F32, P=P)
    g = torch.Generator().manual_seed(1)
    T = 400
    h = torch.randn(T, 24, generator=g).to(BF16).float()
    h2 = h.clone()
    h2[3] = -h2[3]
    c = cfg["layers"][0]["mixer"]
    ref, ref2 = (R.delta_mixer(Pd, "l0.mix.", c, x.double(), 1e-5) for x in (h, h2))
    assert rel(ref[-20:], ref2[-20:]) > 1e-3            # the far token matters at the end
    for x, r in ((h, ref), (h2, ref2)):
        assert rel(_mixer_in_portions(op, cache, x, F32, [250, 100] + [1] * 50), r) < 2e-5


# the bf16 runs of the kv_rank 64 / 128 / 256 rows take the matrix-core kernel, everything else the vector-ALU one
ATTN_SIZES = [(3, 16, 8, 16, 24, 12, None), (5, 12, 6, 10, 9, 5, 4), (1, 8, 4, 8, 8, 1, 0), (4, 32, 16, 32, 64, None, None),
              (2, 16, 8, 24, 40, 70, None), (6, 48, 32, 40, 64, 33, None), (5, 16, 8, 16, 128, 20, 6), (16, 8, 24, 8, 256, 47, None),
              (1, 16, 16, 16, 64, 3, None), (20, 8, 8, 8, 64, None, None)]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H,D,Rd,V,L,window,rot_dims", ATTN_SIZES)
def test_latent_attention_whole_portions_and_window(dtype, H, D, Rd, V, L, window, rot_dims):
    cfg = R.make_config([R.attention_layer(heads=H, dim=D, rot_dim=Rd, vdim=V, kv_rank=L, window=window, rot_dims=rot_dims, base=500.0)], width=24)
    op, cache, P = _operator(cfg, 6, dtype)
    g = torch.Generator().manual_seed(8)
    T = 90
    h = torch.randn(T, 24, generator=g).to(BF16).float()
    ref = R.latent_attention(P, "l0.mix.", cfg["layers"][0]["mixer"], h.double(), cfg["norm"]["eps"])
    tol = 2e-5 if dtype == F32 else 3e-2
    for sizes in ([T], [1] * T, [2] * 45, [7, 1, 30, 2, 50], [89, 1]):
        assert rel(_mixer_in_portions(op, cache, h, dtype, sizes), ref) < tol, sizes
    op.KEYS_PER_SPLIT = op.MFMA_KEYS_PER_SPLIT = 4               # several workgroups share a token's keys and are merged
    try:
        assert rel(_mixer_in_portions(op, cache, h, dtype, [60] + [1] * 30), ref) < tol
        assert rel(_mixer_in_portions(op, cache, h, dtype, [33, 57]), ref) < tol
    finally:
        del op.KEYS_PER_SPLIT, op.MFMA_KEYS_PER_SPLIT
    if dtype == BF16:                   # both kernels, the same cache rows: they differ by the rounding of the weights alone
        from ktransformers_amd._native_hyb import latattn_mfma_eligible
        took_matrix_cores = latattn_mfma_eligible(op._config(cache))
        assert took_matrix_cores == (L in (64, 128, 256, 512))
        a = _mixer_in_portions(op, cache, h, dtype, [50, 40])
        op.USE_MATRIX_CORES = False
        try:
            b = _mixer_in_portions(op, cache, h, dtype, [50, 40])
        finally:
            del op.USE_MATRIX_CORES
        assert rel(a, b) < (1.5e-2 if took_matrix_cores else 1e-7)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("L", [8, 64])
@pytest.mark.parametrize("window,query,back", [(16, 40, 15), (16, 40, 16), (16, 15, 15), (16, 16, 16), (8, 8, 7), (8, 8, 8), (33, 64, 32),
                                               (33, 64, 33), (5, 4, 4), (1, 9, 0), (1, 9, 1), (40, 100, 39), (40, 100, 40)])
def test_one_key_at_the_window_edge_stands_out(dtype, window, query, back, L):
    """The rotated key part is not normed: a token whose input is scaled up gets a score far above all others, so the query `back`
    positions after it takes its value alone when it is inside the window (back < window) and must not see it when it is one place
    outside.  Page size 8: the key sits at, before and after page borders.  As a prompt, and with the query decoded alone."""
    cfg = R.make_config([R.attention_layer(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=L, window=window, rot_dims=0, scale=1.0)], width=24)
    P = R.random_checkpoint(cfg, 9)
    P["l0.mix.sink"] = torch.full((2,), -30.0).to(BF16)
    op, cache, Pd = _operator(cfg, 9, dtype, P=P)
    g = torch.Generator().manual_seed(window * 100 + query)
    T = query + 3
    h = torch.randn(T, 24, generator=g).to(BF16).float() * 0.3
    key = query - back
    c = cfg["layers"][0]["mixer"]
    # sign of the boosted key's rotated score for the query (rot_dims = 0: no dependence on the positions)
    qr = (h[query].double() @ Pd["l0.mix.q"].T).view(2, 16)[:, 8:]
    kr = h[key].double() @ Pd["l0.mix.dkv"].T[:, L:]
    if back > 0:
        h[key] = h[key] * (60.0 if float((qr @ kr).sum()) > 0 else -60.0)
    ref = R.latent_attention(Pd, "l0.mix.", c, h.double(), 1e-5)
    if 0 < back < window:        # the case is what it claims: without the boosted key the answer is another
        h0 = h.clone()
        h0[key] = 0.0
        assert rel(R.latent_attention(Pd, "l0.mix.", c, h0.double(), 1e-5)[query], ref[query]) > 0.05
    tol = 2e-5 if dtype == F32 else 4e-2
    for sizes in ([T], [query] + [1] * 3, [2] * (T // 2) + [1] * (T % 2)):
        got = _mixer_in_portions(op, cache, h, dtype, sizes)
        assert rel(got[query], ref[query]) < tol and rel(got, ref) < tol, sizes


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("E,top,F,SF,T", [(6, 2, 24, 24, 50), (3, 1, 7, 0, 9), (4, 4, 32, 64, 130), (16, 3, 40, 8, 1), (3, 2, 136, 16, 400),
                                          (5, 2, 20, 0, 333)])
def test_mixture_of_experts(dtype, E, top, F, SF, T):
    cfg = R.make_config([R.delta_layer(mlp=R.moe_mlp(experts=E, top=top, ff=F, shared_ff=SF, scale=1.3))], width=40)
    model, cache, P = build(cfg, 4, dtype)
    g = torch.Generator().manual_seed(3)
    h = torch.randn(T, 40, generator=g).to(BF16).float()
    ref = R.moe_ff(P, "l0.mlp.", cfg["layers"][0]["mlp"], h.double())
    shared, rider, rows, pos, tw = model.l0.mlp(h.to(dtype).to(DEV))
    got = (rows[pos.long()].view(T, top, -1) * tw.unsqueeze(-1)).sum(1) + (shared if shared is not None else 0.0)
    assert rider is None and rel(got, ref) < (2e-5 if dtype == F32 else 2e-2)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_poly_norm_feed_forward(dtype):
    cfg = R.make_config([R.delta_layer(mlp=R.dense_mlp(ff=37))], width=40)
    model, cache, P = build(cfg, 4, dtype)
    h = torch.randn(11, 40, generator=torch.Generator().manual_seed(3)).to(BF16).float()
    y, rider = model.l0.mlp(h.to(dtype).to(DEV))
    assert rel(y + model.l0.mlp.down_bias, R.dense_ff(P, "l0.mlp.", h.double(), 1e-5)) < (2e-5 if dtype == F32 else 2e-2)


# ---- the model through the framework --------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(dtype, name):
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 11, dtype)
    toks = tokens_of(cfg, 50, 1)
    ref, ref_layers = R.forward(P, cfg, toks, return_layers=True)
    cache.admit("a")
    fb = cache.plan([("a", len(toks))])
    logits, layers = model(torch.tensor(toks, dtype=torch.int32, device=DEV), None, cache, batch=fb, return_layers=True)
    assert layers.shape == ref_layers.shape
    for li in range(ref_layers.shape[0]):
        assert rel(layers[li], ref_layers[li]) < TOL[dtype], f"layer run {li}"
    assert rows_close(logits, ref, dtype)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("name", ["loop", "odd"])
def test_prefill_equals_token_by_token_and_portions(dtype, name):
    cfg = CONFIGS[name]()
    model, cache, P = build(cfg, 12, dtype, page_size=8)
    eng = engine_of(model, cache)
    toks = tokens_of(cfg, 41, 2)
    ref = R.forward(P, cfg, toks)
    whole = steps(eng, "w", toks, [41])
    assert rows_close(whole, ref, dtype)
    for sizes in ([1] * 41, [2] * 20 + [1], [3, 5, 8, 9, 16], [39, 2], [7] + [1] * 34):
        got = steps(eng, "p", toks, sizes)
        assert rows_close(got, ref, dtype), sizes
        assert rows_close(got, whole, dtype, f32_tol=2e-5), sizes      # cutting the prompt changes rounding only
    assert not cache.requests and len(cache.free_pages) == cache.num_pages


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_unequal_batch_equals_each_alone_and_reuses_pages_and_slots(dtype):
    cfg = CONFIGS["loop"]()
    model, cache, P = build(cfg, 13, dtype, max_tokens=400, max_requests=3, page_size=8)
    eng = engine_of(model, cache)
    reqs = {"a": tokens_of(cfg, 1, 3), "b": tokens_of(cfg, 37, 4), "c": tokens_of(cfg, 90, 5)}
    tail = 6
    alone = {rid: R.forward(P, cfg, toks + tokens_of(cfg, tail, 50 + len(toks))) for rid, toks in reqs.items()}
    for round_ in range(3):       # every round takes the pages and slots the previous one gave back, in another order
        order = list(reqs)[round_:] + list(reqs)[:round_]
        lg = eng.step([{"id": r, "tokens": reqs[r], "want": [len(reqs[r]) - 1]} for r in order])
        got, ref = [lg], [torch.stack([alone[r][len(reqs[r]) - 1] for r in order])]
        live = list(order)
        for step in range(tail):
            ext = {r: tokens_of(cfg, tail, 50 + len(reqs[r]))[step] for r in live}
            ending = [r for r in live if (r == "a" and step == 1) or step == tail - 1]       # the short request leaves early
            lg = eng.step([{"id": r, "tokens": [ext[r]], "want": [0]} for r in live], ending)
            got.append(lg)
            ref.append(torch.stack([alone[r][len(reqs[r]) + step] for r in live]))
            live = [r for r in live if r not in ending]
        assert rows_close(torch.cat(got), torch.cat(ref), dtype), round_
        assert not cache.requests


def test_long_decoding_past_windows_and_pages():
    cfg = CONFIGS["loop"]()
    model, cache, P = build(cfg, 14, F32, page_size=16)
    eng = engine_of(model, cache)
    toks = tokens_of(cfg, 150, 6)
    ref = R.forward(P, cfg, toks)
    got = [eng.step([{"id": "d", "tokens": toks[:10], "want": [9]}])]
    for t in range(10, len(toks)):
        got.append(eng.step([{"id": "d", "tokens": [toks[t]], "want": [0]}]))
    assert rows_rel(torch.cat(got), ref[9:]) < TOL[F32]


def test_cache_grows_beyond_its_first_size():
    cfg = CONFIGS["loop"]()
    model, cache, P = build(cfg, 15, F32, max_tokens=32, max_requests=1, page_size=8)
    eng = engine_of(model, cache)
    reqs = {k: tokens_of(cfg, 30 + 7 * k, k) for k in range(4)}          # more requests and tokens than the cache was made for
    lg = eng.step([{"id": k, "tokens": t, "want": [len(t) - 1]} for k, t in reqs.items()])
    for i, (k, t) in enumerate(reqs.items()):
        assert rows_rel(lg[i:i + 1], R.forward(P, cfg, t)[-1:]) < TOL[F32]
    lg = eng.step([{"id": k, "tokens": [5], "want": [0]} for k in reqs])  # and the state survived the re-allocation
    for i, (k, t) in enumerate(reqs.items()):
        assert rows_rel(lg[i:i + 1], R.forward(P, cfg, t + [5])[-1:]) < TOL[F32]


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_greedy_generation_through_both_loops(dtype):
    """util.generate.prefill_and_generate (one request, chunked prefill, the decode step replayed from a captured HIP graph) and
    BatchEngine.generate (a batch of unequal prompts) against the plain statement's greedy continuation."""
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.models.modeling_pilavik import pilavik_layer_specs
    from ktransformers_amd.util.generate import prefill_and_generate
    cfg = CONFIGS["loop"]()
    model, cache, P = build(cfg, 16, dtype, page_size=16)
    prompts = {"p": tokens_of(cfg, 19, 7), "q": tokens_of(cfg, 5, 8)}
    n_new = 12
    out = engine_of(model, cache).generate(prompts, max_new_tokens=n_new)
    for rid, prompt in prompts.items():
        assert len(out[rid]) == n_new
        lg = R.forward(P, cfg, prompt + out[rid])
        for k, tok in enumerate(out[rid]):      # teacher-forced on the framework's own tokens: the argmax wherever its margin is clear
            row = lg[len(prompt) - 1 + k]
            top2 = row.topk(2).values
            if float(top2[0] - top2[1]) > (1e-3 if dtype == F32 else 0.25):
                assert tok == int(row.argmax()), (rid, k)
    for use_graph in (False, True):
        c1 = KHybridCache(pilavik_layer_specs(model.config), 256, max_requests=1, page_size=16, dtype=dtype, device=DEV)
        ids = torch.tensor([prompts["p"]], dtype=torch.int64, device=DEV)
        toks = prefill_and_generate(model, ids, c1, max_new_tokens=n_new, use_cuda_graph=use_graph, chunk_size=8).tolist()
        assert toks == out["p"], (use_graph, toks, out["p"])


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps of a batch replayed from a captured HIP graph, with eager work (another request's prompt) and a change of the
    batch between replays: every replay against the eager engine's logits and against the plain statement."""
    cfg = CONFIGS["wide"]()
    model, cache, P = build(cfg, 21, dtype, page_size=16)
    _, cache2, _ = build(cfg, 21, dtype, page_size=16)
    eager, graphed = engine_of(model, cache2), engine_of(model, cache, use_graph=True)
    reqs = {"a": tokens_of(cfg, 30, 1), "b": tokens_of(cfg, 9, 2)}
    cont = {r: tokens_of(cfg, 12, 30 + i) for i, r in enumerate(reqs)}
    ref = {r: R.forward(P, cfg, reqs[r] + cont[r]) for r in reqs}
    for eng in (eager, graphed):
        eng.step([{"id": r, "tokens": t, "want": []} for r, t in reqs.items()])
    live, got, want = list(reqs), [], []
    for k in range(12):
        entries = [{"id": r, "tokens": [cont[r][k]], "want": [0]} for r in live]
        end = ["b"] if k == 6 else []
        le, lg = eager.step(entries, end), graphed.step(entries, end)
        assert rows_rel(lg, le) < (1e-5 if dtype == F32 else 2e-2), k
        got.append(lg)
        want.append(torch.stack([ref[r][len(reqs[r]) + k] for r in live]))
        live = [r for r in live if r not in end]
        if k == 3:      # eager work between two replays
            for eng in (eager, graphed):
                eng.step([{"id": "c", "tokens": tokens_of(cfg, 20, 9), "want": [19]}], ["c"])
    assert rows_close(torch.cat(got), torch.cat(want), dtype)
    assert len(graphed._graphs) >= 2
