"""Host side of the Pilavik family, no GPU: the plain statement's own consistency (the delta rule carried token by token, the window's
edges, the sink, the order of layer runs), config reading, the registry, rule injection on the meta device, and the cache / state
manager's per-run caches and slots."""
import os

import pytest
import torch

from oracle import pilavik_ref as R


def test_statement_is_causal_and_the_window_has_the_edges_it_says():
    cfg = R.make_config([R.attention_layer(heads=2, window=4)])
    P = R.as_double(R.random_checkpoint(cfg, 1))
    c = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(0)
    h = torch.randn(12, 32, generator=g).double()
    full = R.latent_attention(P, "l0.mix.", c, h, 1e-5)
    assert torch.allclose(R.latent_attention(P, "l0.mix.", c, h[:7], 1e-5), full[:7], atol=1e-12)       # later tokens change nothing
    h2 = h.clone()
    h2[5] += 1.0                         # position 5 is seen by 5 .. 8 (window 4) and by nobody else
    moved = (R.latent_attention(P, "l0.mix.", c, h2, 1e-5) - full).abs().amax(-1) > 1e-9
    assert moved.tolist() == [False] * 5 + [True] * 4 + [False] * 3
    # the sink takes weight and gives nothing: raising it shrinks the output towards zero, a very low one leaves a plain softmax
    P2 = dict(P)
    P2["l0.mix.sink"] = P["l0.mix.sink"] + 50.0
    assert R.latent_attention(P2, "l0.mix.", c, h, 1e-5).abs().max() < 1e-12
    # a rotation turns pairs (2i, 2i + 1) and nothing behind `dims`
    x = torch.arange(6, dtype=torch.float64).view(1, 6) + 1
    y = R.rotate_pairs(x, torch.tensor([3]), 100.0, 4)
    assert torch.equal(y[0, 4:], x[0, 4:]) and abs(float(y[0, 0]) - (1 * torch.cos(torch.tensor(3.0)) - 2 * torch.sin(torch.tensor(3.0))).item()) < 1e-7
    assert abs(float(y[0, 3]) - (4 * torch.cos(torch.tensor(0.3, dtype=torch.float64)) + 3 * torch.sin(torch.tensor(0.3, dtype=torch.float64))).item()) < 1e-12


def test_delta_rule_reads_what_it_has_just_written():
    cfg = R.make_config([R.delta_layer(heads=1, kv_heads=1, dim=4, vdim=3, conv=1)], width=8)
    P = R.as_double(R.random_checkpoint(cfg, 2))
    h = torch.randn(1, 8, generator=torch.Generator().manual_seed(0)).double()
    # one token from an empty memory: S = k (beta v)^T, o = S^T q = beta v (k . q) — not zero
    out = R.delta_mixer(P, "l0.mix.", cfg["layers"][0]["mixer"], h, 1e-5)
    assert out.abs().max() > 1e-6
    conv = R.short_conv(torch.tensor([[1.0], [10.0], [100.0]]), torch.tensor([[0.5, 2.0, 3.0]]))
    assert conv[:, 0].tolist() == [3.0, 32.0, 320.5]           # last column = the current token, zeros before the start


def test_order_of_layer_runs():
    from ktransformers_amd.models.modeling_pilavik import layer_runs
    assert layer_runs(4, None) == [(0, None), (1, None), (2, None), (3, None)]
    assert layer_runs(4, {"start": 1, "stop": 3, "times": 2}) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert layer_runs(2, {"start": 0, "stop": 2, "times": 3}) == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    assert [(i, t if first else None) for i, t, first in R.layer_runs({"layers": [0] * 4, "loop": {"start": 1, "stop": 3, "times": 2}})] == \
        layer_runs(4, {"start": 1, "stop": 3, "times": 2})


def test_config_reader_checks_and_registry():
    from ktransformers_amd.models import MODEL_REGISTRY, architecture_of
    from ktransformers_amd.models.modeling_pilavik import make_pilavik_config, pilavik_layer_specs
    raw = R.make_config([R.delta_layer(heads=6, kv_heads=3, dim=10, vdim=9, conv=4), R.attention_layer(kv_rank=20, rot_dim=6)],
                        loop={"start": 0, "stop": 1, "times": 2})
    cfg = make_pilavik_config(raw)
    assert cfg.num_hidden_layers == 2 and cfg.width == raw["width"] and cfg.eps == raw["norm"]["eps"] and len(cfg.runs) == 3
    specs = pilavik_layer_specs(cfg)
    assert specs[0] == specs[1] == {"delta": (6, 10, 9), "conv": (2 * 3 * 10 + 6 * 9, 4)} and specs[2] == {"latent": 26}
    assert architecture_of(raw) == "Pilavik" and torch.float32 in MODEL_REGISTRY["Pilavik"].dtypes
    for breakit, match in ((lambda c: c["layers"][0].update(type="serial"), "layer type"),
                           (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "multiple"),
                           (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "even"),
                           (lambda c: c["layers"][1].update(mlp={"kind": "sparse"}), "feed-forward"),
                           (lambda c: c["loop"].update(stop=5), "loop")):
        bad = R.make_config([R.delta_layer(heads=6, kv_heads=3), R.attention_layer()], loop={"start": 0, "stop": 1, "times": 2})
        breakit(bad)
        with pytest.raises(ValueError, match=match):
            make_pilavik_config(bad)


def test_rules_replace_every_arithmetic_leaf():
    from ktransformers_amd.models import RULES_DIR
    from ktransformers_amd.models.modeling_deepseek import _Leaf
    from ktransformers_amd.models.modeling_pilavik import PilavikForCausalLM, make_pilavik_config
    from ktransformers_amd.optimize.optimize import gen_optimize_config, inject, load_rules
    from ktransformers_amd.util.loader import DictLoader
    raw = R.make_config([R.delta_layer(mlp=R.moe_mlp()), R.attention_layer(mlp=R.dense_mlp()), R.delta_layer()],
                        loop={"start": 0, "stop": 2, "times": 2})
    cfg = make_pilavik_config(raw)
    with torch.device("meta"):
        model = PilavikForCausalLM(cfg)
    plan = {}
    gen_optimize_config(model, plan, load_rules(os.path.join(RULES_DIR, "Pilavik.yaml")))
    inject(model, plan, cfg, DictLoader(R.random_checkpoint(raw, 0)))
    kinds = {n: type(m).__name__ for n, m in model.named_modules() if type(m).__name__.startswith("K")}
    assert kinds["l0.mix"] == "KGatedDeltaMixer" and kinds["l1.mix"] == "KLatentWindowAttention"
    assert kinds["l0.mlp"] == "KSigmoidRoutedMoE" and kinds["l1.mlp"] == "KPolyNormMLP" and "l2.mlp" not in kinds and model.l2.mlp is None
    assert {"embed", "loop", "head", "final.norm", "l0.norm1", "l0.norm1b", "l0.rg1", "l0.rg2", "l1.norm2b"} <= set(kinds)
    left = [n for n, m in model.named_modules() if isinstance(m, _Leaf)]
    assert all(".orig_module" in n for n in left)          # every leaf that is left sits behind its operator


def test_cache_manager_keeps_one_cache_or_state_per_layer_run():
    from ktransformers_amd.models.custom_cache import KHybridCache
    specs = [{"delta": (2, 4, 8), "conv": (24, 3)}, {"latent": 12}, {"delta": (2, 4, 8), "conv": (24, 1)}, {"latent": 12}]
    c = KHybridCache(specs, max_tokens=64, max_requests=2, page_size=8, dtype=torch.float32, device="cpu")
    assert c.S[0].shape == (2, 2, 4, 8) and c.conv[0].shape == (2, 2, 24) and c.conv[2] is None and c.n[0] is None and c.m[0] is None
    assert c.lat_caches[1].shape == (c.num_pages * 8, 12) and c.lat_caches[0] is None and c.S[1] is None
    assert c.lat_caches[1].data_ptr() != c.lat_caches[3].data_ptr()
    assert len(c.state_tensors()) == 3
    c.lat_caches[1][0, 0] = 5.0
    c.conv[0][1, 1, 3] = 2.0
    c.admit("a"), c.admit("b"), c.admit("x")                 # one request more than the cache was made for: slots grow, contents stay
    c.plan([("x", 200)])
    assert c.S[0].shape[0] == c.max_requests >= 3 and c.conv[0].shape[0] == c.max_requests and float(c.conv[0][1, 1, 3]) == 2.0
    assert c.lat_caches[3].shape[0] == c.num_pages * 8 and float(c.lat_caches[1][0, 0]) == 5.0
    with pytest.raises(ValueError):
        KHybridCache([{"rec": (1, 2, 2), "delta": (1, 2, 2)}], 8, dtype=torch.float32, device="cpu")
