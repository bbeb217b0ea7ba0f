"""Host side of the Mitotar family, no GPU: the plain statement's own consistency (token-by-token recurrence = carried state, the
attention's causality and head-mixing linearity), config reading, the registry, rule injection on the meta device, the cache /
state manager's page and slot bookkeeping, and the step function's batching with a stand-in model."""
import os

import pytest
import torch

from oracle import mitotar_ref as R


def test_recurrence_carries_state_across_portions():
    g = torch.Generator().manual_seed(0)
    T, N, D, V = 23, 2, 5, 7
    q, k = torch.randn(T, N, D, generator=g).double(), torch.randn(T, N, D, generator=g).double()
    v = torch.randn(T, N, V, generator=g).double()
    i, f = torch.randn(T, N, generator=g).double(), -torch.rand(T, N, generator=g).double()
    whole, final = R.mlstm_recurrence(q, k, v, i, f)
    for cut in (1, 2, 11, 22):
        a, st = R.mlstm_recurrence(q[:cut], k[:cut], v[:cut], i[:cut], f[:cut])
        b, st2 = R.mlstm_recurrence(q[cut:], k[cut:], v[cut:], i[cut:], f[cut:], state=st)
        assert torch.allclose(torch.cat([a, b]), whole, atol=1e-12)
        assert all(torch.allclose(x, y, atol=1e-12) for x, y in zip(st2, final))
    # the running maximum starts at 0, not at minus infinity: a strongly negative first input gate must not be renormalised away
    o, (_, _, m) = R.mlstm_recurrence(q[:1], k[:1], v[:1], torch.full((1, N), -9.0).double(), torch.full((1, N), -0.1).double())
    assert torch.allclose(m, torch.full((N,), -0.1).double())


def test_attention_is_causal_unnormalised_and_linear_in_the_mixing_matrix():
    cfg = R.make_config(width=32, heads=4, kv_heads=2, dim=8, n_layers=1)
    P = {k: v.double() for k, v in R.random_checkpoint(cfg, 3).items()}
    c = cfg["layers"][0]["mixer"]["left"]
    g = torch.Generator().manual_seed(1)
    h = torch.randn(12, 32, generator=g).double()
    full = R.sigmoid_talk_attention(P, "l0.mix.left", c, h, 1e-5)
    assert torch.allclose(R.sigmoid_talk_attention(P, "l0.mix.left", c, h[:7], 1e-5), full[:7], atol=1e-12)      # later tokens change nothing
    P2 = dict(P)
    P2["l0.mix.left.talk"] = 2 * P["l0.mix.left.talk"]
    assert torch.allclose(R.sigmoid_talk_attention(P2, "l0.mix.left", c, h, 1e-5), 2 * full, atol=1e-12)        # no normalisation over keys
    assert abs(R.distance_slopes(8)[0].item() - 0.5) < 1e-15 and abs(R.distance_slopes(8)[7].item() - 2.0 ** -8) < 1e-15
    assert R.query_temperature(torch.tensor([0, 62, 63, 127]), 0.5, 64).tolist() == pytest.approx([1.0, 1.0, 1 + 0.5 * 0.6931471805599453] * 1 + [1 + 0.5 * 1.0986122886681098])


def test_config_reader_checks_and_registry():
    from ktransformers_amd.models import MODEL_REGISTRY, architecture_of
    from ktransformers_amd.models.modeling_mitotar import make_mitotar_config, mitotar_layer_specs
    raw = R.make_config(n_layers=3, mlp_none_at=(1,), heads=6, kv_heads=3, dim=10, r_heads=2, r_dim=4, r_vdim=9)
    cfg = make_mitotar_config(raw)
    assert cfg.num_hidden_layers == 3 and cfg.width == raw["width"] and cfg.eps == raw["norm"]["eps"]
    assert mitotar_layer_specs(cfg)[0] == {"attn": (3, 10), "rec": (2, 4, 9)}
    assert architecture_of(raw) == "Mitotar" and torch.float32 in MODEL_REGISTRY["Mitotar"].dtypes
    assert architecture_of({"architectures": ["DeepseekV3ForCausalLM"]}) == "DeepseekV3ForCausalLM"
    with pytest.raises(KeyError):
        architecture_of({"architecture": "nothing"})
    bad = R.make_config()
    bad["layers"][0]["mixer"]["left"]["vdim"] += 1
    with pytest.raises(ValueError, match="vdim"):
        make_mitotar_config(bad)
    bad = R.make_config()
    bad["layers"][1]["type"] = "serial"
    with pytest.raises(ValueError, match="layer type"):
        make_mitotar_config(bad)
    bad = R.make_config(heads=4, kv_heads=3)
    with pytest.raises(ValueError, match="multiple"):
        make_mitotar_config(bad)


def test_rules_replace_every_arithmetic_leaf():
    from ktransformers_amd.models import RULES_DIR
    from ktransformers_amd.models.modeling_deepseek import _Leaf
    from ktransformers_amd.models.modeling_mitotar import MitotarForCausalLM, make_mitotar_config
    from ktransformers_amd.optimize.optimize import gen_optimize_config, inject, load_rules
    from ktransformers_amd.util.loader import DictLoader
    raw = R.make_config(n_layers=2, mlp_none_at=(0,))
    cfg = make_mitotar_config(raw)
    with torch.device("meta"):
        model = MitotarForCausalLM(cfg)
    plan = {}
    gen_optimize_config(model, plan, load_rules(os.path.join(RULES_DIR, "Mitotar.yaml")))
    inject(model, plan, cfg, DictLoader(R.random_checkpoint(raw, 0)))
    left = [n for n, m in model.named_modules() if isinstance(m, _Leaf)]
    wrapped = {n for n, m in model.named_modules() if type(m).__name__.startswith("K")}
    assert {"embed", "head", "final.norm", "l0.mix", "l0.norm1", "l1.mlp", "l1.norm2"} <= wrapped
    assert "l0.mlp" not in wrapped and model.l0.mlp is None
    assert all(".orig_module" in n for n in left)          # every leaf that is left sits behind its operator


def test_cache_manager_pages_and_slots():
    from ktransformers_amd.models.custom_cache import KHybridCache
    c = KHybridCache([{"attn": (2, 8), "rec": (2, 4, 8)}, {"attn": (1, 4), "rec": None}], max_tokens=64, max_requests=2, page_size=8,
                     dtype=torch.float32, device="cpu")
    assert c.k_caches[1].shape == (c.num_pages * 8, 1, 4) and c.S[1] is None and c.S[0].shape == (2, 2, 4, 8)
    c.admit("a"), c.admit("b")
    fb = c.plan([("a", 9), ("b", 3)])
    assert fb.q_indptr.tolist() == [0, 9, 12] and fb.pos0.tolist() == [0, 0] and fb.positions.tolist() == list(range(9)) + [0, 1, 2]
    pa = c.requests["a"]["pages"]
    assert len(pa) == 2 and fb.cache_loc.tolist()[:9] == [pa[0] * 8 + i for i in range(8)] + [pa[1] * 8]
    assert fb.page_indptr.tolist() == [0, 2, 3] and fb.page_indices.tolist() == pa + c.requests["b"]["pages"]
    fb = c.plan([("b", 1), ("a", 1)])                       # decode step, other order
    assert fb.positions.tolist() == [3, 9] and fb.pos0.tolist() == [3, 9] and fb.slot.tolist() == [c.requests["b"]["slot"], c.requests["a"]["slot"]]
    with pytest.raises(KeyError):
        c.admit("a")
    free_before, slot_a = len(c.free_pages), c.requests["a"]["slot"]
    c.release("a")
    assert len(c.free_pages) == free_before + 2
    c.admit("n")                                            # the freed slot and pages are handed out again
    assert c.requests["n"]["slot"] == slot_a
    c.plan([("n", 8)])
    assert c.requests["n"]["pages"][0] in pa
    # more requests and tokens than the cache was sized for: it grows, old contents stay in front
    c.k_caches[0][0, 0, 0] = 5.0
    gen = c.generation
    c.admit("x")
    c.plan([("x", 200)])
    assert c.generation > gen and c.max_requests >= 3 and float(c.k_caches[0][0, 0, 0]) == 5.0 and c.S[0].shape[0] == c.max_requests
    assert c.live_tokens() == 4 + 8 + 200
    c.reset()
    assert not c.requests and len(c.free_pages) == c.num_pages and len(c.free_slots) == c.max_requests


def test_step_function_batches_and_releases():
    from ktransformers_amd.models.custom_cache import KHybridCache
    from ktransformers_amd.util.batch_engine import BatchEngine
    calls = []

    def fake_model(ids, pos, cache, batch=None, logits_rows=None):
        calls.append((ids.tolist(), batch.q_indptr.tolist(), batch.positions.tolist(), logits_rows.tolist()))
        return torch.arange(len(logits_rows) * 3, dtype=torch.float32).view(-1, 3)

    cache = KHybridCache([{"attn": (1, 4), "rec": (1, 2, 2)}], 64, max_requests=2, page_size=4, dtype=torch.float32, device="cpu")
    eng = BatchEngine(fake_model, cache)
    out = eng.step([{"id": "a", "tokens": [5, 6, 7], "want": [0, 2]}, {"id": "b", "tokens": [9], "want": []}])
    assert out.shape == (2, 3) and calls[-1] == ([5, 6, 7, 9], [0, 3, 4], [0, 1, 2, 0], [0, 2])
    out = eng.step([{"id": "a", "tokens": [1], "want": []}, {"id": "b", "tokens": [2], "want": []}], end=["b"])
    assert out is None and calls[-1][2] == [3, 1] and "b" not in cache.requests and "a" in cache.requests
    with pytest.raises(IndexError):
        eng.step([{"id": "a", "tokens": [1], "want": [1]}])
    with pytest.raises(ValueError):
        eng.step([{"id": "c", "tokens": [], "want": []}])


def test_trace_runner_is_executable_and_documents_itself():
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    assert os.access(path, os.X_OK)
    text = open(path).read()
    assert "BatchEngine" in text and "load_model" in text
