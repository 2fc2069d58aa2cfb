"""Prefill and decode throughput of Loluzen beside the closest existing model of equal layer sizes
(bench.py --loluzen): a dense Llama (grouped-query attention, one feed-forward per layer).

Both models are random-init bf16 and run through the same engine and the same measurement as
bench/dofivik_bench.py: prefill is ONE step of `prompts` x `prompt_len` tokens, decode is `decode_batch`
sequences at context `context` generating greedily (HIP-graph steps, sampling included).
"""
from __future__ import annotations

import importlib.util
import json
import os


def loluzen_layers(n_layers, heads, kv, dim, rot, l_heads, l_kv, r_heads, r_dim, r_vdim, ff):
    att = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "conv": 4,
           "rot": {"base": 500000.0, "dims": rot,
                   "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    par = {"left": {"heads": l_heads, "kv_heads": l_kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5},
           "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim}}
    return [{"type": "attention" if i % 2 == 0 else "parallel", "mixer": dict(att if i % 2 == 0 else par),
             "mlp": {"kind": "dense", "ff": ff}} for i in range(n_layers)]


SIZES = {
    # name: width, layers, vocab, loluzen mixer sizes, llama (heads, kv heads, head dim, ff)
    "1b-class": dict(width=2048, layers=8, vocab=32000,
                     lol=dict(heads=32, kv=8, dim=64, rot=32, l_heads=16, l_kv=2, r_heads=16, r_dim=64, r_vdim=128,
                              ff=8192),
                     llama=dict(heads=32, kv=8, hd=64, ff=8192)),
    "8b-class": dict(width=4096, layers=4, vocab=32000,
                     lol=dict(heads=32, kv=8, dim=128, rot=64, l_heads=16, l_kv=2, r_heads=32, r_dim=64, r_vdim=128,
                              ff=14336),
                     llama=dict(heads=32, kv=8, hd=128, ff=14336)),
}


def run(a) -> int:
    import torch
    from xgserve.models import build_model
    from xgserve.models.config import ModelConfig, loluzen_config
    if not torch.cuda.is_available():
        print("bench.py --loluzen needs a GPU")
        return 2
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("dofivik_bench", os.path.join(here, "dofivik_bench.py"))
    common = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(common)
    dev = torch.device("cuda", 0)
    results = []
    for name in a.loluzen_sizes.split(","):
        s = SIZES[name]
        zcfg = loluzen_config(f"loluzen-{name}", s["width"], s["vocab"], loluzen_layers(s["layers"], **s["lol"]),
                              embed_scale=s["width"] ** 0.5, residual_mult=0.5, max_position=16384)
        ll = s["llama"]
        lcfg = ModelConfig(f"llama-{name}", "llama", s["width"], s["layers"], ll["heads"], ll["kv"], ll["hd"], ll["ff"],
                           s["vocab"], 16384, 500000.0)
        row = {"size": name, "width": s["width"], "layers": s["layers"], "prompts": a.dofivik_prompts,
               "prompt_len": a.prompt_len, "decode_batch": a.concurrency, "context": a.dofivik_context}
        for key, cfg in (("loluzen", zcfg), ("llama", lcfg)):
            if a.loluzen_only and key != a.loluzen_only:
                continue
            model = build_model(cfg, device=dev)
            row[key] = common.measure(model, dev, a.dofivik_prompts, a.prompt_len, a.concurrency, a.dofivik_context,
                                      a.steps, a.warmup)
            del model
            torch.cuda.empty_cache()
        results.append(row)
    print(json.dumps({"metric": "loluzen_vs_llama_tokens_per_sec", "dtype": "bf16",
                      "data": "synthetic (random-token prompts, random-init weights)", "results": results}), flush=True)
    return 0
