"""Dofivik on the engine against the dense fp64 oracle (tests/dofivik_oracle.py).

Every test runs on the CPU (PyTorch forms of the ops, same scheduler / cache / state code) and,
marked `gpu`, on the HIP kernels in float32 and bfloat16. Configurations and weights are made
here; the oracle shares no code with xgserve.
"""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import dofivik_oracle as orc
from xgserve.engine import EngineConfig, LLMEngine, SamplingParams
from xgserve.models import build_model, get_config
from xgserve.models.config import dofivik_config
from xgserve.ops import seqmix as sq

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64

CASES = [pytest.param("cpu", "float32", id="cpu-f32"),
         pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def _att(heads, dim, rot, vdim, R, Rq, win, base, scale, **kw):
    return dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, kv_rank=R, q_rank=Rq, scale=scale,
                mask={"size": win}, rot={"base": base, "dims": rot}, **kw)


def config_a():
    """Delta layer first, attention without feed-forward, a shared cache with other head counts."""
    a1 = _att(3, 20, 12, 28, 40, 36, 9, 500.0, 0.21)
    a2 = _att(5, 16, 12, 8, 40, 24, 13, 500.0, 0.3, kv_from=1)
    return {"architecture": "Dofivik", "width": 96, "vocab": 160, "postln_alpha": 1.7, "canon": {"taps": 4},
            "norm": {"eps": 1e-5},
            "layers": [{"type": "general_delta", "mixer": {"heads": 3, "dim": 24}, "mlp": {"kind": "dense", "ff": 80}},
                       {"type": "latent_attention", "mixer": a1, "mlp": None},
                       {"type": "latent_attention", "mixer": a2, "mlp": {"kind": "dense", "ff": 56}},
                       {"type": "general_delta", "mixer": {"heads": 2, "dim": 40}, "mlp": None}]}


def config_b():
    """One head, a window of one token, two taps, equal ranks: values that are easily confused."""
    a1 = _att(1, 8, 8, 8, 16, 16, 1, 10.0, 1.0)
    a2 = _att(2, 12, 4, 12, 24, 8, 70, 10000.0, 0.4)
    return {"architecture": "Dofivik", "width": 48, "vocab": 97, "postln_alpha": 1.0, "canon": {"taps": 2},
            "norm": {"eps": 1e-6},
            "layers": [{"type": "latent_attention", "mixer": a1, "mlp": {"kind": "dense", "ff": 48}},
                       {"type": "general_delta", "mixer": {"heads": 1, "dim": 16}, "mlp": {"kind": "dense", "ff": 32}},
                       {"type": "latent_attention", "mixer": a2, "mlp": None}]}


_MADE = {}


def made(name, tmp_path_factory):
    """(config, oracle weights, checkpoint dir) of a test model, written once per session."""
    if name not in _MADE:
        cfg = {"a": config_a, "b": config_b}[name]()
        Wt = orc.random_weights(cfg, seed=7 if name == "a" else 11, decay_rank=5 if name == "a" else 3)
        path = str(tmp_path_factory.mktemp("dofivik_" + name))
        orc.write_checkpoint(path, cfg, Wt)
        _MADE[name] = (cfg, Wt, path)
    return _MADE[name]


def engine(path, device, dtype, **kw):
    args = dict(model=path, checkpoint=path, device=device, dtype=dtype, block_size=4, num_blocks=64, max_num_seqs=3,
                max_num_batched_tokens=256, max_model_len=200, use_graphs=False)
    args.update(kw)
    return LLMEngine(EngineConfig(**args))


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def rel_err(got, ref):
    got, ref = got.detach().to("cpu", F64), ref.to(F64)
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    r = ref - ref.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt()).max())


def run_portions(eng, rid, toks, portions):
    """Feed `toks` in the given portion sizes (the rest one by one); logits of every position."""
    out, at = [], 0
    sizes = list(portions)
    while at < len(toks):
        n = sizes.pop(0) if sizes else 1
        n = min(n, len(toks) - at)
        end = [rid] if at + n == len(toks) else []
        out.append(eng.score_step([(rid, toks[at:at + n], list(range(n)))], end))
        at += n
    return torch.cat(out, 0)


# ---------------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompt_matches_oracle(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 45, 1)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = eng.score_step([("w", toks, list(range(len(toks))))], ["w"])
    assert rel_err(got, ref) < TOL[dtype]
    assert eng.sched.num_used_blocks() == 0


@pytest.mark.parametrize("device,dtype", CASES)
def test_residual_after_every_layer(device, dtype, tmp_path_factory):
    cfg, Wt, path = made("a", tmp_path_factory)
    toks = tokens_of(cfg, 17, 2)
    res = []
    orc.forward(cfg, Wt, toks, res)
    m = build_model(get_config(path), device=device, dtype=getattr(torch, dtype), checkpoint=path)
    eng = LLMEngine(EngineConfig(model=path, device=device, dtype=dtype, block_size=4, num_blocks=16, max_num_seqs=2,
                                 max_model_len=64, use_graphs=False), model=m)
    seen = []
    hooks = [L.register_forward_hook(lambda mod, i, o: seen.append(o.detach().to("cpu", F64).clone())) for L in m.layers]
    eng.score_step([("x", toks, [0])], ["x"])
    for h in hooks:
        h.remove()
    tol = 1e-4 if dtype == "float32" else 5e-2
    for got, ref in zip(seen, res):
        assert float((got - ref).abs().max()) < tol * float(ref.abs().max())


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_decode_token_by_token_equals_prefill(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 40, 3)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "d", toks, [])
    assert rel_err(got, ref) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("portions", [[2, 2, 3, 2, 9, 1, 1, 5, 2], [7, 1, 13, 2], [33, 2], [1, 2, 4, 8, 16]])
def test_portions_of_any_size(portions, device, dtype, tmp_path_factory):
    cfg, Wt, path = made("a", tmp_path_factory)
    toks = tokens_of(cfg, 42, 4)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "p", toks, portions)
    assert rel_err(got, ref) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decoding_past_the_window(device, dtype, tmp_path_factory):
    cfg, Wt, path = made("b", tmp_path_factory)  # windows 1 and 70, positions up to 170
    toks = tokens_of(cfg, 170, 5)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "l", toks, [9])
    assert rel_err(got, ref) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_reused_pages_and_slots(device, dtype, tmp_path_factory):
    """Unequal requests share steps (portions beside single tokens), sit steps out, end, and later ones take
    over their slots and pages: two slots and a pool that holds only the live requests."""
    cfg, Wt, path = made("a", tmp_path_factory)
    lens = {"r0": 23, "r1": 9, "r2": 31, "r3": 1, "r4": 14}
    toks = {k: tokens_of(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: orc.forward(cfg, Wt, v) for k, v in toks.items()}
    eng = engine(path, device, dtype, num_blocks=14, max_num_seqs=2)
    # (request, tokens) per step
    steps = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 3)], [("r1", 4)], [("r0", 9)], [("r2", 6), ("r0", 1)],
             [("r0", 7), ("r2", 1)], [("r2", 2)], [("r3", 1), ("r2", 13)], [("r4", 3), ("r2", 1)], [("r2", 8), ("r4", 1)],
             [("r4", 10)]]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for st in steps:
        entries, end = [], []
        for k, n in st:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                end.append(k)
        lg = eng.score_step(entries, end)
        o = 0
        for k, n in st:
            got[k].append(lg[o:o + n])
            o += n
    assert at == lens
    for k in lens:
        assert rel_err(torch.cat(got[k], 0), ref[k]) < TOL[dtype], k
    assert eng.sched.num_used_blocks() == 0 and eng.sched.num_running() == 0


@pytest.mark.parametrize("device,dtype", CASES)
def test_batch_rows_equal_alone(device, dtype, tmp_path_factory):
    cfg, Wt, path = made("b", tmp_path_factory)
    a, b, c = tokens_of(cfg, 30, 20), tokens_of(cfg, 5, 21), tokens_of(cfg, 12, 22)
    eng = engine(path, device, dtype)
    alone = [eng.score_step([(n, t, list(range(len(t))))], [n]) for n, t in (("a", a), ("b", b), ("c", c))]
    both = eng.score_step([("a", a, list(range(30))), ("b", b, list(range(5))), ("c", c, list(range(12)))], ["a", "b", "c"])
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert rel_err(both[:30], alone[0].cpu()) < tol and rel_err(both[30:35], alone[1].cpu()) < tol
    assert rel_err(both[35:], alone[2].cpu()) < tol


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_scheduler(device, dtype, tmp_path_factory):
    """add_request / step with the engine's own scheduler (chunked prompts, several requests at once; HIP graphs
    on the GPU): every generated token is the oracle's argmax on the same history, up to rounding."""
    cfg, Wt, path = made("a", tmp_path_factory)
    prompts = [tokens_of(cfg, n, 30 + i) for i, n in enumerate((19, 3, 11, 1))]
    eng = engine(path, device, dtype, max_num_batched_tokens=8, max_num_seqs=3, use_graphs=True,
                 graph_batch_sizes=[1, 2, 4])
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [12] * 4
    for p, o in zip(prompts, outs):
        ref = orc.forward(cfg, Wt, p + o[:-1])
        for i, tok in enumerate(o):
            row = ref[len(p) - 1 + i]
            gap = float(row.max() - row[tok])
            assert gap <= (1e-3 if dtype == "float32" else 0.15) * float(row.std()), (len(p), i, tok, int(row.argmax()))
    assert eng.sched.num_used_blocks() == 0


def test_trace_runner_cli(tmp_path, tmp_path_factory):
    cfg, Wt, path = made("b", tmp_path_factory)
    a, b = tokens_of(cfg, 21, 40), tokens_of(cfg, 6, 41)
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [0, 9]}, {"id": "b", "tokens": b[:2], "want": []}],
              "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:], "want": [10]}], "end": ["a"]}]
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(x) for x in lines) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    V = cfg["vocab"]
    ra, rb = orc.forward(cfg, Wt, a), orc.forward(cfg, Wt, b)
    g0 = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(-1, V))
    g1 = torch.from_numpy(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(-1, V))
    assert rel_err(g0, ra[[0, 9]]) < 2e-4 and rel_err(g1, rb[[5]]) < 2e-4 and rel_err(g2, ra[[20]]) < 2e-4


def test_config_rejects_what_the_design_does_not_have():
    cfg = config_a()
    bad = copy.deepcopy(cfg["layers"])
    bad[1]["mixer"]["kv_from"] = 2  # a later layer
    with pytest.raises(ValueError):
        dofivik_config("x", 96, 160, bad)
    bad = copy.deepcopy(cfg["layers"])
    bad[0]["type"] = "something_else"
    with pytest.raises(ValueError):
        dofivik_config("x", 96, 160, bad)
    with pytest.raises(ValueError):
        LLMEngine(EngineConfig(model="dofivik-tiny", device="cpu", num_blocks=8, max_num_seqs=2, max_model_len=32,
                               use_graphs=False, draft_model="llama-tiny-draft", num_speculative_tokens=2))


# ---------------------------------------------------------------------------------- mechanisms alone
OP_CASES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


def seq_meta(device, rows, block_size, tables):
    """rows: [(slot, context length, tokens in this step)] -> SeqMeta; tables: page list per row."""
    qsl, sl, slots, tseq, pos, smap = [0], [], [], [], [], []
    width = max(len(t) for t in tables)
    for i, (slot, ctx, q) in enumerate(rows):
        qsl.append(qsl[-1] + q)
        sl.append(ctx + q)
        slots.append(slot)
        for p in range(ctx, ctx + q):
            tseq.append(i)
            pos.append(p)
            smap.append(tables[i][p // block_size] * block_size + p % block_size)
    bt = [t + [0] * (width - len(t)) for t in tables]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return sq.SeqMeta(len(rows), max(r[2] for r in rows), i32(qsl), i32(sl), i32(slots), i32(bt), i32(tseq), i32(pos),
                      i32(smap))


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_conv_carries_inputs_across_portions(device, taps):
    g = torch.Generator().manual_seed(taps)
    C, lens = 70, [150, 11, 1]
    xs = [torch.randn(n, C, generator=g) for n in lens]
    w = torch.randn(C, taps, generator=g)
    refs = [orc.shifted_conv(x.to(F64), w.to(F64)) for x in xs]
    state = torch.full((4, taps - 1, C), 1e3, device=device)  # stale values a new sequence must not read
    slots = [2, 0, 3]
    cuts = [[1, 2, 1, 70, 3, 66, 7], [4, 2, 2, 3], [1]]
    got = [[] for _ in lens]
    at = [0, 0, 0]
    while any(c for c in cuts):
        rows, parts, who = [], [], []
        for i in range(3):
            if cuts[i]:
                q = cuts[i].pop(0)
                rows.append((slots[i], at[i], q))
                parts.append(xs[i][at[i]:at[i] + q])
                who.append((i, q))
                at[i] += q
        sm = seq_meta(device, rows, 4, [[0] * 64 for _ in rows])
        y = sq.causal_conv_residual(torch.cat(parts).to(device).contiguous(), w.to(device), state, sm, torch.float32)
        o = 0
        for i, q in who:
            got[i].append(y[o:o + q].cpu())
            o += q
    for i in range(3):
        assert torch.allclose(torch.cat(got[i]).to(F64), refs[i], atol=1e-4), i


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("W", [77, 96, 2304])
def test_norm_after_scaled_sum(device, W):
    g = torch.Generator().manual_seed(0)
    x, y = torch.randn(9, W, generator=g), torch.randn(9, W, generator=g)
    b, w = torch.randn(W, generator=g), torch.randn(W, generator=g) * 0.2
    ref = orc.unit_rms(1.9 * x.to(F64) + y.to(F64) + b.to(F64), 1e-5) * (1 + w.to(F64))
    xd = x.clone().to(device)
    out = sq.scaled_add_rmsnorm(xd, y.to(device), w.to(device), 1e-5, 1.9, b.to(device), 1.0)
    assert out.data_ptr() == xd.data_ptr() and torch.allclose(out.cpu().to(F64), ref, atol=1e-5)
    out = sq.scaled_add_rmsnorm(x.to(device), None, w.to(device), 1e-5, 1.0, None, 1.0, inplace=False,
                                out_dtype=torch.float32)
    assert torch.allclose(out.cpu().to(F64), orc.unit_rms(x.to(F64), 1e-5) * (1 + w.to(F64)), atol=1e-5)


@pytest.mark.parametrize("device", OP_CASES)
def test_xielu_both_branches(device):
    z = torch.linspace(-30, 6, 4001).reshape(1, -1)
    b = torch.full((4001,), 0.25)
    p, q = 0.3, -0.8
    ref = orc.xielu(z.to(F64) + 0.25, p, q)
    sp, cn = math.log1p(math.exp(p)), 0.5 + math.log1p(math.exp(q))
    got = sq.xielu(z.to(device), b.to(device), sp, cn)
    assert torch.allclose(got.cpu().to(F64), ref, rtol=1e-5, atol=1e-5)


def latent_reference(qabs, qrot, lat, key, gate, window, scale):
    """Dense fp64 softmax over [max(0, i - window + 1), i] in latent space; qrot / key already rotated."""
    H, T, R = qabs.shape
    out = torch.zeros(H, T, R, dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1)
        sc = (qabs[:, i] @ lat[lo:i + 1].T + qrot[i] @ key[lo:i + 1].T) * scale
        out[:, i] = (torch.softmax(sc, -1) @ lat[lo:i + 1]) * torch.sigmoid(gate[i])[:, None]
    return out


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(3, 24, 8, 5), (5, 32, 8, 8), (20, 48, 16, 4), (2, 160, 24, 8), (2, 288, 8, 4)],
                         ids=["odd", "r32", "h20", "r160", "r288"])
@pytest.mark.parametrize("window,bs", [(7, 4), (64, 16), (300, 16), (1, 4)])
def test_latent_attention_one_key_stands_out(device, dtype, shape, window, bs):
    """For every query the key exactly `reach` back gets a dominating score, with reach = window - 1 (the
    last one seen), window (the first one not seen), page borders and far keys among hundreds: a window
    that is one token off, or a wrong page, changes the output by O(1). Prompt portion and single tokens.
    The shapes cover the general kernel and the matrix-core one (bf16, latent size a multiple of 16), with
    more heads than one wave's 16 query slots."""
    g = torch.Generator().manual_seed(window)
    H, R, rd, dn = shape
    T = 340
    td = getattr(torch, dtype)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(td).to(F64)  # noqa: E731  (representable in td)
    lat, key_raw, gate = rnd(T, R), rnd(T, rd), rnd(T, H)
    q = (torch.randn(T, H, dn + rd, generator=g) * 0.3).to(td).to(F64)
    qabs = torch.randn(H, T, R, generator=g, dtype=F64) * 0.3
    reaches = [window - 1, window, bs, bs - 1, 2 * bs, 0]
    for i in range(T):
        j = i - reaches[i % len(reaches)]
        if j >= 0:
            qabs[i % H, i] += 9.0 * lat[j] / lat[j].norm()
    qabs = qabs.to(td).to(F64)
    rot = sq.build_rot_table(rd, 100.0, T + 1)
    qrot = orc.rotate_interleaved(q[:, :, dn:], range(T), rd, 100.0)
    # pages in scrambled order; the cache is filled through latent_prep's own write path
    npages = (T + bs - 1) // bs
    perm = torch.randperm(npages + 3, generator=g)[:npages].tolist()
    cache = torch.zeros((npages + 3) * bs, R + rd, device=device, dtype=td)
    proj = torch.cat([rnd(T, 6), lat, key_raw], -1).to(td).to(device)
    ones = torch.ones(R, device=device)
    split = 200  # [0, 200) as one portion, then single tokens
    outs = []
    steps = [(0, split)] + [(t, 1) for t in range(split, T)]
    for ctx, n in steps:
        sm = seq_meta(device, [(0, ctx, n)], bs, [perm])
        sl = slice(ctx, ctx + n)
        sq.latent_prep(proj[sl].contiguous(), 0, 6, 6, R, rd, torch.ones(6, device=device), ones, 0.0, rot.to(device), rd,
                       sm, cache)
        o = sq.latent_attention(qabs[:, sl].to(td).to(device).contiguous(), q[sl].to(td).to(device).contiguous(), dn,
                                gate[sl].to(td).to(device).contiguous(), cache, rot.to(device), rd, window, 0.5, bs, sm)
        outs.append(o.float().cpu())
    got = torch.cat(outs, 1).to(F64)
    # the reference reads what latent_prep stored (normed latent, rotated key), through the page table
    rows = torch.tensor([perm[p // bs] * bs + p % bs for p in range(T)])
    stored = cache.float().cpu().to(F64)[rows]
    f = 1.0 / torch.sqrt((lat * lat).mean(-1, keepdim=True))
    key = orc.rotate_interleaved(key_raw, range(T), rd, 100.0)
    tol = 2e-4 if dtype == "float32" else 4e-2
    assert float((stored[:, :R] - lat * f).abs().max()) < tol and float((stored[:, R:] - key).abs().max()) < tol
    ref = latent_reference(qabs, qrot, stored[:, :R], stored[:, R:], gate, window, 0.5)
    assert float((got - ref).abs().max()) < tol


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("H,D", [(3, 24), (2, 32), (2, 64), (1, 16), (1, 128), (1, 72)])
def test_delta_rule_state_over_portions_and_slots(device, H, D):
    """Head sizes of the one-pass kernel (any size) and of the two-pass one (16 / 32 / 64)."""
    W, eps = 40, 1e-5
    cfg = {"width": W, "vocab": 8, "canon": {"taps": 1}, "layers": [{"type": "general_delta", "mixer": {"heads": H, "dim": D},
                                                                    "mlp": None}]}
    Wt = orc.random_weights(cfg, seed=D, decay_rank=5)
    m = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(3)
    lens = [90, 6]
    hs = [torch.randn(n, W, generator=g, dtype=F64) for n in lens]
    refs = [orc.delta_rule(Wt, "l0.mix.", m, h, eps) for h in hs]
    from xgserve.models.dofivik import DeltaRuleMixer
    mix = DeltaRuleMixer(W, m, 5, eps, device, torch.float32)
    HD = H * D
    for j, n in enumerate(("r", "k", "v", "g", "a")):
        mix.in_proj.data[j * HD:(j + 1) * HD] = Wt["l0.mix." + n].float()
    mix.in_proj.data[5 * HD:] = Wt["l0.mix.w1"].float()
    for dst, n in ((mix.w2, "w2"), (mix.w0, "w0"), (mix.a_bias, "a.b"), (mix.norm, "norm"), (mix.o, "o")):
        dst.data.copy_(Wt["l0.mix." + n].float())
    state = torch.full((3, H, D, D), 50.0, device=device)  # stale state of an earlier owner
    cuts = [[2, 1, 40, 1, 1, 45], [3, 1, 2]]
    slots, at, got = [1, 2], [0, 0], [[], []]
    while any(cuts):
        rows, parts, who = [], [], []
        for i in range(2):
            if cuts[i]:
                q = cuts[i].pop(0)
                rows.append((slots[i], at[i], q))
                parts.append(hs[i][at[i]:at[i] + q])
                who.append((i, q))
                at[i] += q
        sm = seq_meta(device, rows, 4, [[0] * 32 for _ in rows])
        y = mix(torch.cat(parts).float().to(device), sm, state)
        o = 0
        for i, q in who:
            got[i].append(y[o:o + q].cpu())
            o += q
    for i in range(2):
        assert torch.allclose(torch.cat(got[i]).to(F64), refs[i], atol=2e-4, rtol=1e-3), i
