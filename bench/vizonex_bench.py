"""Prefill and decode throughput of Vizonex beside the closest existing models of equal layer sizes
(bench.py --vizonex): a Mixtral-type model (grouped-query attention + routed experts in every layer)
and a dense Llama.

All models are random-init bf16 and run through the same engine and the same measurement as
bench/dofivik_bench.py: prefill is ONE step of `prompts` x `prompt_len` tokens, decode is `decode_batch`
sequences at context `context` generating greedily (HIP-graph steps, sampling included).
"""
from __future__ import annotations

import importlib.util
import json
import os


def vizonex_layers(n_layers, heads, kv, dim, chunk, s_heads, s_vdim, s_state, s_groups, experts, top, e_ff, shared_ff,
                   dense_ff):
    att = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "mask": {"size": chunk}}
    ssm = {"heads": s_heads, "vdim": s_vdim, "state": s_state, "groups": s_groups, "norm_groups": s_groups, "conv": 4}
    moe = {"kind": "moe", "expert": {"ff": e_ff, "limit": 7.0}, "shared": {"ff": shared_ff, "limit": 7.0},
           "router": {"experts": experts, "top": top, "scale": 2.5, "groups": {"count": 4, "keep": 2}}}
    out = []
    for i in range(n_layers):
        mixer = ("attention", att) if i % 2 == 0 else ("mamba2", ssm)
        mlp = {"kind": "dense", "ff": dense_ff} if i == 0 else moe
        out.append({"type": mixer[0], "mixer": dict(mixer[1]), "mlp": mlp})
    return out


SIZES = {
    # name: width, layers, vocab, vizonex sizes, mixtral / llama (heads, kv heads, head dim, expert ff, dense ff)
    "1b-class": dict(width=2048, layers=8, vocab=32000,
                     viz=dict(heads=32, kv=8, dim=64, chunk=1024, s_heads=64, s_vdim=64, s_state=128, s_groups=8,
                              experts=8, top=2, e_ff=2048, shared_ff=2048, dense_ff=8192),
                     ref=dict(heads=32, kv=8, hd=64, e_ff=2048, ff=8192, experts=8, top=2)),
    "8b-class": dict(width=4096, layers=4, vocab=32000,
                     viz=dict(heads=32, kv=8, dim=128, chunk=4096, s_heads=128, s_vdim=64, s_state=128, s_groups=8,
                              experts=8, top=2, e_ff=3584, shared_ff=3584, dense_ff=14336),
                     ref=dict(heads=32, kv=8, hd=128, e_ff=3584, ff=14336, experts=8, top=2)),
}


def run(a) -> int:
    import torch
    from xgserve.models import build_model
    from xgserve.models.config import ModelConfig, vizonex_config
    if not torch.cuda.is_available():
        print("bench.py --vizonex needs a GPU")
        return 2
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("dofivik_bench", os.path.join(here, "dofivik_bench.py"))
    common = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(common)
    dev = torch.device("cuda", 0)
    results = []
    for name in a.vizonex_sizes.split(","):
        s = SIZES[name]
        vcfg = vizonex_config(f"vizonex-{name}", s["width"], s["vocab"], vizonex_layers(s["layers"], **s["viz"]), taps=4,
                              max_position=16384)
        r = s["ref"]
        mcfg = ModelConfig(f"mixtral-{name}", "mixtral", s["width"], s["layers"], r["heads"], r["kv"], r["hd"], r["e_ff"],
                           s["vocab"], 16384, 1000000.0, num_experts=r["experts"], experts_per_token=r["top"])
        lcfg = ModelConfig(f"llama-{name}", "llama", s["width"], s["layers"], r["heads"], r["kv"], r["hd"], r["ff"],
                           s["vocab"], 16384, 500000.0)
        row = {"size": name, "width": s["width"], "layers": s["layers"], "prompts": a.dofivik_prompts,
               "prompt_len": a.prompt_len, "decode_batch": a.concurrency, "context": a.dofivik_context}
        for key, cfg in (("vizonex", vcfg), ("mixtral", mcfg), ("llama", lcfg)):
            if a.vizonex_only and key != a.vizonex_only:
                continue
            model = build_model(cfg, device=dev)
            row[key] = common.measure(model, dev, a.dofivik_prompts, a.prompt_len, a.concurrency, a.dofivik_context,
                                      a.steps, a.warmup)
            del model
            torch.cuda.empty_cache()
        results.append(row)
    print(json.dumps({"metric": "vizonex_vs_mixtral_llama_tokens_per_sec", "dtype": "bf16",
                      "data": "synthetic (random-token prompts, random-init weights)", "results": results}), flush=True)
    return 0
