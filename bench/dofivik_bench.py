"""Prefill and decode throughput of Dofivik beside a Llama of equal layer sizes (bench.py --dofivik).

Both models are random-init bf16 and run through the same engine: prefill is ONE step of
`prompts` x `prompt_len` tokens (the runner's eager path, logits of the last tokens only), decode is
`decode_batch` sequences at context `context` generating greedily (HIP-graph steps, sampling
included). Sizes are layer shapes of real model classes with few layers, so a run takes seconds.
"""
from __future__ import annotations

import json
import time
from dataclasses import replace

import numpy as np


def dofivik_layers(n_layers, heads, dim, rot, vdim, R, Rq, window, ff, d_heads, d_dim):
    att = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": R, "q_rank": Rq,
           "scale": (dim + rot) ** -0.5, "mask": {"size": window}, "rot": {"base": 5e5, "dims": rot}}
    out = []
    for i in range(n_layers):
        if i % 2 == 0:
            out.append({"type": "latent_attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": ff}})
        else:
            out.append({"type": "general_delta", "mixer": {"heads": d_heads, "dim": d_dim}, "mlp": {"kind": "dense", "ff": ff}})
    return out


SIZES = {
    # name: (width, layers, vocab, dofivik mixer sizes, llama (heads, kv heads, head dim, ff))
    "1b-class": dict(width=2048, layers=8, vocab=32000,
                     dof=dict(heads=32, dim=64, rot=32, vdim=64, R=256, Rq=768, window=1024, ff=8192, d_heads=32, d_dim=64),
                     llama=dict(heads=32, kv=8, hd=64, ff=8192)),
    "8b-class": dict(width=4096, layers=4, vocab=32000,
                     dof=dict(heads=32, dim=128, rot=64, vdim=128, R=512, Rq=1536, window=4096, ff=14336, d_heads=64,
                              d_dim=64),
                     llama=dict(heads=32, kv=8, hd=128, ff=14336)),
}


def _engine(model, dev, max_len, batch, tokens):
    from xgserve.engine import EngineConfig, LLMEngine
    blocks = (batch + 2) * ((max_len + 15) // 16 + 1)
    return LLMEngine(EngineConfig(model=model.cfg.name, device=str(dev), max_num_seqs=batch, num_blocks=blocks,
                                  max_num_batched_tokens=tokens, max_model_len=max_len, use_graphs=True,
                                  enable_prefix_cache=False, graph_batch_sizes=[batch], async_schedule=True),
                     model=model)


def measure(model, dev, prompts, prompt_len, decode_batch, context, steps, warmup):
    import torch
    from xgserve.engine import SamplingParams
    V = model.cfg.vocab_size
    rng = np.random.default_rng(0)
    max_len = max(prompt_len, context + steps + warmup + 8) + 16
    eng = _engine(model, dev, max_len, max(decode_batch, prompts), max(prompts * prompt_len, 2048))
    out = {"params": int(sum(p.numel() for p in model.parameters()))}
    # ---- prefill: one step of prompts x prompt_len tokens
    times = []
    for it in range(3):
        ent = [(f"p{it}-{i}", rng.integers(5, V - 5, size=prompt_len).tolist(), [prompt_len - 1]) for i in range(prompts)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.score_step(ent, [e[0] for e in ent])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    out["prefill_tokens_per_s"] = round(prompts * prompt_len / min(times[1:]), 1)
    out["prefill_ms"] = round(1000 * min(times[1:]), 3)
    # ---- decode: decode_batch sequences at `context`, greedy, graph steps
    for i in range(decode_batch):
        eng.add_request(f"d{i}", rng.integers(5, V - 5, size=context).tolist(),
                        SamplingParams(max_tokens=steps + warmup + 4, temperature=0.0, ignore_eos=True))
    n = 0
    while eng.stats_counters["decode_steps"] < warmup and n < 10_000:
        eng.step()
        n += 1
    torch.cuda.synchronize()
    g0, t0 = eng.stats_counters["generation_tokens"], time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    out["decode_tokens_per_s"] = round((eng.stats_counters["generation_tokens"] - g0) / dt, 1)
    out["decode_ms_per_step"] = round(1000 * dt / steps, 4)
    for i in range(decode_batch):
        eng.abort(f"d{i}")
    del eng
    torch.cuda.empty_cache()
    return out


def run(a) -> int:
    import torch
    from xgserve.models import build_model
    from xgserve.models.config import ModelConfig, dofivik_config
    if not torch.cuda.is_available():
        print("bench.py --dofivik needs a GPU")
        return 2
    dev = torch.device("cuda", 0)
    results = []
    for name in a.dofivik_sizes.split(","):
        s = SIZES[name]
        d = s["dof"]
        dcfg = dofivik_config(f"dofivik-{name}", s["width"], s["vocab"],
                              dofivik_layers(s["layers"], d["heads"], d["dim"], d["rot"], d["vdim"], d["R"], d["Rq"],
                                             d["window"], d["ff"], d["d_heads"], d["d_dim"]),
                              postln_alpha=2.0, taps=4, max_position=16384)
        ll = s["llama"]
        lcfg = ModelConfig(f"llama-{name}", "llama", s["width"], s["layers"], ll["heads"], ll["kv"], ll["hd"], ll["ff"],
                           s["vocab"], 16384, 500000.0)
        row = {"size": name, "width": s["width"], "layers": s["layers"], "prompts": a.dofivik_prompts,
               "prompt_len": a.prompt_len, "decode_batch": a.concurrency, "context": a.dofivik_context}
        for key, cfg in (("dofivik", dcfg), ("llama", lcfg)):
            if a.dofivik_only and key != a.dofivik_only:
                continue
            model = build_model(cfg, device=dev)
            row[key] = measure(model, dev, a.dofivik_prompts, a.prompt_len, a.concurrency, a.dofivik_context, a.steps,
                               a.warmup)
            del model
            torch.cuda.empty_cache()
        results.append(row)
    print(json.dumps({"metric": "dofivik_vs_llama_tokens_per_sec", "dtype": "bf16",
                      "data": "synthetic (random-token prompts, random-init weights)", "results": results}), flush=True)
    return 0
