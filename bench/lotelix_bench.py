"""Prefill and decode throughput of Lotelix beside the closest existing models of equal layer sizes
(bench.py --lotelix): a Mixtral-type model (grouped-query attention + routed experts in every layer)
and a dense Llama.

All models are random-init bf16 and run through the same engine and the same measurement as
bench/dofivik_bench.py: prefill is ONE step of `prompts` x `prompt_len` tokens, decode is `decode_batch`
sequences at context `context` generating greedily (HIP-graph steps, sampling included).
"""
from __future__ import annotations

import importlib.util
import json
import os


def lotelix_layers(n_layers, heads, kv, dim, window, gru, l_heads, l_kv, r_heads, r_dim, r_vdim, experts, top, e_ff):
    rot = {"base": 500000.0, "dims": dim, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    att = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "mask": {"size": window},
           "rot": rot, "v_mix": True}
    par = {"left": {"heads": l_heads, "kv_heads": l_kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
                    "rot": {"base": 1000000.0, "dims": dim}},
           "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": 16.0, "decay_rank": 16}}
    moe = {"kind": "moe", "expert": {"ff": e_ff}, "router": {"experts": experts, "top": top}}
    kinds = [("attention", att), ("mingru", {"width": gru}), ("attention", att), ("parallel", par)]
    return [{"type": kinds[i % 4][0], "mixer": dict(kinds[i % 4][1]), "mlp": dict(moe)} for i in range(n_layers)]


SIZES = {
    # name: width, layers, vocab, lotelix sizes, mixtral / llama (heads, kv heads, head dim, expert ff, dense ff)
    "1b-class": dict(width=2048, layers=8, vocab=32000,
                     lot=dict(heads=32, kv=8, dim=64, window=1024, gru=2048, l_heads=16, l_kv=4, r_heads=16, r_dim=64,
                              r_vdim=128, experts=8, top=2, e_ff=2048),
                     ref=dict(heads=32, kv=8, hd=64, e_ff=2048, ff=8192, experts=8, top=2)),
    "8b-class": dict(width=4096, layers=4, vocab=32000,
                     lot=dict(heads=32, kv=8, dim=128, window=4096, gru=4096, l_heads=16, l_kv=4, r_heads=32, r_dim=64,
                              r_vdim=128, experts=8, top=2, e_ff=3584),
                     ref=dict(heads=32, kv=8, hd=128, e_ff=3584, ff=14336, experts=8, top=2)),
}


def run(a) -> int:
    import torch
    from xgserve.models import build_model
    from xgserve.models.config import ModelConfig, lotelix_config
    if not torch.cuda.is_available():
        print("bench.py --lotelix needs a GPU")
        return 2
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("dofivik_bench", os.path.join(here, "dofivik_bench.py"))
    common = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(common)
    dev = torch.device("cuda", 0)
    results = []
    for name in a.lotelix_sizes.split(","):
        s = SIZES[name]
        xcfg = lotelix_config(f"lotelix-{name}", s["width"], s["vocab"], lotelix_layers(s["layers"], **s["lot"]),
                              embed_scale=s["width"] ** 0.5, norm_groups=2, max_position=16384)
        r = s["ref"]
        mcfg = ModelConfig(f"mixtral-{name}", "mixtral", s["width"], s["layers"], r["heads"], r["kv"], r["hd"], r["e_ff"],
                           s["vocab"], 16384, 1000000.0, num_experts=r["experts"], experts_per_token=r["top"])
        lcfg = ModelConfig(f"llama-{name}", "llama", s["width"], s["layers"], r["heads"], r["kv"], r["hd"], r["ff"],
                           s["vocab"], 16384, 500000.0)
        row = {"size": name, "width": s["width"], "layers": s["layers"], "prompts": a.dofivik_prompts,
               "prompt_len": a.prompt_len, "decode_batch": a.concurrency, "context": a.dofivik_context}
        for key, cfg in (("lotelix", xcfg), ("mixtral", mcfg), ("llama", lcfg)):
            if a.lotelix_only and key != a.lotelix_only:
                continue
            model = build_model(cfg, device=dev)
            row[key] = common.measure(model, dev, a.dofivik_prompts, a.prompt_len, a.concurrency, a.dofivik_context,
                                      a.steps, a.warmup)
            del model
            torch.cuda.empty_cache()
        results.append(row)
    print(json.dumps({"metric": "lotelix_vs_mixtral_llama_tokens_per_sec", "dtype": "bf16",
                      "data": "synthetic (random-token prompts, random-init weights)", "results": results}), flush=True)
    return 0
