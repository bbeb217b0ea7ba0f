"""Command-line generation for any registered model family — the role of the reference's local_chat.py (archive/ktransformers/
local_chat.py:60-180: pick the model class by the checkpoint's config, inject the optimize rules, load, then prefill_and_generate),
on token ids since no tokenizer ships with a bare checkpoint folder.

    python -m ktransformers_amd.local_chat --model_path DIR --prompt_ids 5,17,3 [--prompt_ids 9,9 ...] --max_new_tokens 32
                                           [--dtype bfloat16|float32] [--do_sample --temperature T --top_k K --top_p P --seed S]

One --prompt_ids runs util.generate.prefill_and_generate (chunked prefill, the decode step replayed from a captured HIP graph);
several run as one batch through util.batch_engine.BatchEngine (families whose cache is a KHybridCache).  Prints one JSON line
{"request": [generated ids]}."""
from __future__ import annotations

import argparse
import json
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model_path", required=True, help="folder with config.json and *.safetensors")
    ap.add_argument("--prompt_ids", action="append", required=True, help="comma-separated token ids; repeat for a batch")
    ap.add_argument("--max_new_tokens", type=int, default=32)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--optimize_config_path", default=None, help="rule file (default: the family's own)")
    ap.add_argument("--chunk_size", type=int, default=8192)
    ap.add_argument("--no_graph", action="store_true")
    ap.add_argument("--do_sample", action="store_true")
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top_k", type=int, default=0)
    ap.add_argument("--top_p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--device", default="cuda:0")
    a = ap.parse_args(argv)

    import torch
    from ktransformers_amd.models import load_model
    from ktransformers_amd.models.custom_cache import KHybridCache

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids]
    model, config, entry = load_model(a.model_path, dtype=dtype, device=a.device, rule_file=a.optimize_config_path)
    need = sum(len(p) for p in prompts) + len(prompts) * a.max_new_tokens
    cache = entry.make_cache(config, need + 64, max(len(prompts), 1), dtype, a.device)
    gen = torch.Generator(device=a.device).manual_seed(a.seed) if a.do_sample else None
    sampling = dict(do_sample=a.do_sample, temperature=a.temperature, top_k=a.top_k, top_p=a.top_p, generator=gen)
    if len(prompts) == 1:
        from ktransformers_amd.util.generate import prefill_and_generate
        ids = torch.tensor([prompts[0]], dtype=torch.int64, device=a.device)
        out = {"0": prefill_and_generate(model, ids, cache, max_new_tokens=a.max_new_tokens, use_cuda_graph=not a.no_graph,
                                         chunk_size=a.chunk_size, **sampling).tolist()}
    else:
        if not isinstance(cache, KHybridCache):
            raise SystemExit("batched generation from the command line needs a family served through KHybridCache; give one --prompt_ids")
        from ktransformers_amd.util.batch_engine import BatchEngine
        out = BatchEngine(model, cache, use_graph=not a.no_graph).generate({str(i): p for i, p in enumerate(prompts)},
                                                                           max_new_tokens=a.max_new_tokens, **sampling)
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
