"""Vizonex on the engine against the dense fp64 oracle (tests/vizonex_oracle.py).

Every test runs on the CPU (PyTorch forms of the ops, same scheduler / cache / state code) and,
marked `gpu`, on the HIP kernels in float32 and bfloat16. Configurations and weights are made
here; the oracle shares no code with xgserve.
"""
import copy
import json
import os
import subprocess
import sys

import pytest
import torch

import vizonex_oracle as orc
from xgserve.engine import EngineConfig, LLMEngine, SamplingParams
from xgserve.models import build_model, get_config
from xgserve.models.config import vizonex_config
from xgserve.models.seq_cache import LayerCache
from xgserve.ops import seqmix as sq

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64

CASES = [pytest.param("cpu", "float32", id="cpu-f32"),
         pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]
OP_CASES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def _moe(E, count, keep, top, ff, limit, scale, shared):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "shared": shared,
            "router": {"experts": E, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


def config_a():
    """State-space layer first; key size unlike value size; three query heads per key head; groups = heads;
    one norm group; experts without a shared one; a block without feed-forward."""
    att = {"heads": 6, "kv_heads": 2, "dim": 20, "vdim": 12, "scale": 0.31, "mask": {"size": 10}}
    ssm = {"heads": 3, "vdim": 12, "state": 20, "groups": 3, "norm_groups": 1, "conv": 2}
    ssm2 = {"heads": 4, "vdim": 20, "state": 6, "groups": 1, "norm_groups": 4, "conv": 5}
    return {"architecture": "Vizonex", "width": 88, "vocab": 150, "canon": {"taps": 3}, "norm": {"eps": 1e-5},
            "max_positions": 256,
            "layers": [{"type": "mamba2", "mixer": ssm, "mlp": {"kind": "dense", "ff": 72}},
                       {"type": "attention", "mixer": att, "mlp": _moe(6, 3, 2, 3, 24, 1.0, 0.8, None)},
                       {"type": "mamba2", "mixer": ssm2, "mlp": None},
                       {"type": "attention", "mixer": dict(att, mask={"size": 37}, kv_heads=6),
                        "mlp": _moe(12, 2, 1, 2, 16, 0.7, 2.5, {"ff": 40, "limit": 0.9})}]}


def config_b():
    """One head, a chunk of one token, two taps, one expert chosen, one group, groups of one expert."""
    a1 = {"heads": 1, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 1.0, "mask": {"size": 1}}
    a2 = {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.5, "mask": {"size": 64}}
    ssm = {"heads": 1, "vdim": 16, "state": 16, "groups": 1, "norm_groups": 1, "conv": 1}
    return {"architecture": "Vizonex", "width": 48, "vocab": 97, "canon": {"taps": 2}, "norm": {"eps": 1e-6},
            "max_positions": 200,
            "layers": [{"type": "attention", "mixer": a1, "mlp": _moe(4, 1, 1, 1, 32, 5.0, 1.0, {"ff": 16, "limit": 5.0})},
                       {"type": "mamba2", "mixer": ssm, "mlp": _moe(5, 5, 2, 2, 8, 1.5, 1.0, None)},
                       {"type": "attention", "mixer": a2, "mlp": {"kind": "dense", "ff": 40}}]}


_MADE = {}


def made(name, tmp_path_factory):
    """(config, oracle weights, checkpoint dir) of a test model, written once per session."""
    if name not in _MADE:
        cfg = {"a": config_a, "b": config_b}[name]()
        Wt = orc.random_weights(cfg, seed=5 if name == "a" else 13)
        path = str(tmp_path_factory.mktemp("vizonex_" + name))
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


def row_errs(got, ref):
    got, ref = got.detach().to("cpu", F64), ref.to(F64)
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    r = ref - ref.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt()


def close(got, ref, dtype):
    """float32: every position within 2e-4. bfloat16: rounding can tip a router's close call at a token (another
    expert there, felt by the tokens after it through the state), so a few positions may exceed the rounding
    level, none by much; a wrong mechanism is caught by the float32 runs and moves most positions."""
    e = row_errs(got, ref)
    if dtype == "float32":
        return float(e.max()) < TOL[dtype]
    return float((e > TOL[dtype]).double().mean()) <= 0.15 and float(e.max()) < 0.3


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
    assert close(got, ref, dtype)
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
    hooks = [L.register_forward_hook(lambda mod, i, o: seen.append(o[0].detach().to("cpu", F64).clone())) for L in m.layers]
    eng.score_step([("x", toks, [0])], ["x"])
    for h in hooks:
        h.remove()
    tol = 1e-4 if dtype == "float32" else 5e-2
    assert len(seen) == len(res)
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
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("portions", [[2, 2, 3, 2, 9, 1, 1, 5, 2], [7, 1, 13, 2], [33, 2], [1, 2, 4, 8, 16]])
def test_portions_of_any_size(portions, device, dtype, tmp_path_factory):
    cfg, Wt, path = made("a", tmp_path_factory)
    toks = tokens_of(cfg, 42, 4)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "p", toks, portions)
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decoding_over_chunk_edges(device, dtype, tmp_path_factory):
    cfg, Wt, path = made("b", tmp_path_factory)  # chunks of 1 and 64 tokens, positions up to 170
    toks = tokens_of(cfg, 170, 5)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "l", toks, [9])
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_reused_pages_and_slots(device, dtype, tmp_path_factory):
    """Unequal requests share steps (portions beside single tokens), sit steps out, end, and later ones take
    over their slots and pages: two slots and a pool that holds only the live requests."""
    cfg, Wt, path = made("a", tmp_path_factory)
    lens = {"r0": 23, "r1": 9, "r2": 31, "r3": 1, "r4": 14}
    toks = {k: tokens_of(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: orc.forward(cfg, Wt, v) for k, v in toks.items()}
    eng = engine(path, device, dtype, num_blocks=14, max_num_seqs=2)
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
        assert close(torch.cat(got[k], 0), ref[k], dtype), k
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


def test_registered_tiny_model_generates():
    eng = LLMEngine(EngineConfig(model="vizonex-tiny", device="cpu", dtype="float32", block_size=4, num_blocks=32,
                                 max_num_seqs=2, max_model_len=64, use_graphs=False))
    outs = eng.generate([[1, 2, 3, 4, 5], [7]], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [6, 6]


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


def test_save_and_reload_checkpoint(tmp_path):
    from xgserve.models import save_checkpoint
    m = build_model(get_config("vizonex-tiny"), device="cpu", dtype=torch.float32, seed=3)
    save_checkpoint(m, str(tmp_path / "ck"))
    m2 = build_model(get_config(str(tmp_path / "ck")), device="cpu", dtype=torch.float32, checkpoint=str(tmp_path / "ck"))
    for (n1, p1), (n2, p2) in zip(m.named_parameters(), m2.named_parameters()):
        assert n1 == n2 and torch.equal(p1.to(torch.bfloat16).float(), p2), n1


def test_config_rejects_what_the_design_does_not_have():
    cfg = config_a()
    for edit in (lambda L: L[0].__setitem__("type", "something_else"),
                 lambda L: L[1]["mixer"].__setitem__("kv_heads", 4),           # 6 heads do not divide over 4
                 lambda L: L[1]["mlp"]["router"]["groups"].__setitem__("count", 4),   # 6 experts, 4 groups
                 lambda L: L[1]["mlp"]["router"].__setitem__("top", 5),        # more than the kept groups hold
                 lambda L: L[0]["mlp"].__setitem__("kind", "other"),
                 lambda L: L[2]["mixer"].__setitem__("norm_groups", 3)):
        bad = copy.deepcopy(cfg["layers"])
        edit(bad)
        with pytest.raises(ValueError):
            vizonex_config("x", 88, 150, bad)
    with pytest.raises(ValueError):
        LLMEngine(EngineConfig(model="vizonex-tiny", device="cpu", num_blocks=8, max_num_seqs=2, max_model_len=32,
                               use_graphs=False, draft_model="llama-tiny-draft", num_speculative_tokens=2))


# ---------------------------------------------------------------------------------- mechanisms alone
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


def in_portions(device, xs, cuts, slots, fn):
    """Run fn(rows of this step [n, C] on `device`, SeqMeta) over several sequences cut into portions that
    share steps; returns each sequence's outputs in order."""
    got, at = [[] for _ in xs], [0] * len(xs)
    cuts = [list(c) for c in cuts]
    while any(cuts):
        rows, parts, who = [], [], []
        for i in range(len(xs)):
            if cuts[i]:
                q = cuts[i].pop(0)
                rows.append((slots[i], at[i], q))
                parts.append(xs[i][at[i]:at[i] + q])
                who.append((i, q))
                at[i] += q
        sm = seq_meta(device, rows, 4, [[0] * 64 for _ in rows])
        y = fn(torch.cat(parts).to(device), sm)
        o = 0
        for i, q in who:
            got[i].append(y[o:o + q].float().cpu())
            o += q
    return [torch.cat(g).to(F64) for g in got]


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("taps,residual,silu", [(1, False, False), (2, True, False), (4, False, True), (5, True, True)])
def test_conv_with_bias_and_activation_over_portions(device, taps, residual, silu):
    """A strided column block of a wider row, bias, optional residual and silu; stale state in the slots."""
    g = torch.Generator().manual_seed(taps)
    C, lens = 70, [150, 11, 1]
    xs = [torch.randn(n, C + 9, generator=g) for n in lens]
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    refs = []
    for x in xs:
        col = x[:, 5:5 + C].to(F64)
        r = orc.shifted_conv(col, w.to(F64), b.to(F64)) + (col if residual else 0)
        refs.append(orc.silu(r) if silu else r)
    state = torch.full((4, taps - 1, C), 1e3, device=device)
    got = in_portions(device, xs, [[1, 2, 1, 70, 3, 66, 7], [4, 2, 2, 3], [1]], [2, 0, 3],
                      lambda x, sm: sq.causal_conv(x[:, 5:5 + C], w.to(device), b.to(device), state, sm, torch.float32,
                                                   residual=residual, silu=silu))
    for i in range(3):
        assert torch.allclose(got[i], refs[i], atol=1e-4), i


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("W", [77, 96, 2304])
def test_residual_sum_with_scales_and_next_norm(device, W):
    g = torch.Generator().manual_seed(W)
    x, y1, y2, y3 = (torch.randn(9, W, generator=g) for _ in range(4))
    a1, a2, nw = (torch.randn(W, generator=g) for _ in range(3))
    d = lambda t: t.to(device)  # noqa: E731
    ref_x = x.to(F64) + a1.to(F64) * y1.to(F64) + a2.to(F64) * (y2.to(F64) + y3.to(F64))
    xd = d(x.clone())
    n32, nact = sq.residual_norm(xd, d(y1), d(a1), d(y2), d(y3), d(a2), d(nw), 1e-5, torch.float32, True)
    assert torch.allclose(xd.cpu().to(F64), ref_x, atol=1e-5)
    ref_n = orc.unit_rms(ref_x, 1e-5) * nw.to(F64)
    assert torch.allclose(n32.cpu().to(F64), ref_n, atol=1e-5) and torch.allclose(nact.cpu().to(F64), ref_n, atol=1e-5)
    # no feed-forward, no scales, no norm: only the sum
    xd = d(x.clone())
    assert sq.residual_norm(xd, d(y1), None, None, None, None, None, 1e-5) == (None, None)
    assert torch.allclose(xd.cpu(), x + y1, atol=1e-6)
    # nothing to add: the norm alone (the first block's)
    xd = d(x.clone())
    n32, _ = sq.residual_norm(xd, None, None, None, None, None, d(nw), 1e-5, None, True)
    assert torch.equal(xd.cpu(), x) and torch.allclose(n32.cpu().to(F64), orc.unit_rms(x.to(F64), 1e-5) * nw.to(F64), atol=1e-5)


@pytest.mark.parametrize("device", OP_CASES)
def test_embedding_adds_the_position_row(device):
    g = torch.Generator().manual_seed(0)
    tab, pos = torch.randn(11, 24, generator=g), torch.randn(7, 24, generator=g)
    ids = torch.tensor([3, 10, 0, 3], dtype=torch.int32)
    p = torch.tensor([6, 0, 2, 2], dtype=torch.int32)
    got = sq.embed_rows(ids.to(device), tab.to(device), pos.to(device), p.to(device))
    assert torch.allclose(got.cpu(), tab[ids.long()] + pos[p.long()], atol=1e-6)


def _attention_case(device, dtype, H, G, dk, dv, size, bs, T, split, use_sink=True):
    """One key per query gets a dominating score: the first key of the query's chunk (just inside), the
    last key of the chunk before (just outside: must not be seen), keys at page borders, far keys, the
    query itself. A chunk edge that is one token off, or a wrong page, changes the output by O(1)."""
    g = torch.Generator().manual_seed(size * 7 + H)
    td = getattr(torch, dtype)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(td).to(F64)  # noqa: E731  (representable in td)
    k, v = rnd(T, G, dk), rnd(T, G, dv)
    q = torch.randn(T, H, dk, generator=g, dtype=F64) * 0.3
    rep = H // G
    for i in range(T):
        lo = (i // size) * size
        j = [lo, lo - 1, i - bs, i - bs + 1, lo + (i - lo) // 2, i, max(0, i - 150)][i % 7]
        if 0 <= j <= i:
            h = i % H
            q[i, h] += 9.0 * k[j, h // rep] / k[j, h // rep].norm()
    q = q.to(td).to(F64)
    temp = (torch.rand(H, generator=g) + 0.5).to(F64)
    sink = (torch.randn(H, generator=g) * 2 + 2).to(F64)
    scale = 0.7
    ref = orc.chunk_softmax(q, k, v, size, scale, temp, sink if use_sink else torch.full((H,), -1e30, dtype=F64))
    npages = (T + bs - 1) // bs
    perm = torch.randperm(npages + 3, generator=g)[:npages].tolist()
    kc = torch.zeros((npages + 3) * bs, G * dk, device=device, dtype=td)
    vc = torch.zeros((npages + 3) * bs, G * dv, device=device, dtype=td)
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], -1).to(td).to(device)
    outs = []
    for ctx, n in [(0, split)] + [(t, 1) for t in range(split, T)]:
        sm = seq_meta(device, [(0, ctx, n)], bs, [perm])
        qq = sq.qk_norm_cache(proj[ctx:ctx + n].contiguous(), H * dk, G * dk, G * dv, None, None, 0.0, sm, kc, vc)
        o = sq.masked_attention(qq, kc, vc, H, G, dk, dv, sq.MASK_CHUNK, size, scale, temp.float().to(device),
                                sink.float().to(device) if use_sink else None, bs, sm)
        outs.append(o.float().cpu())
    got = torch.cat(outs, 0).to(F64).reshape(T, H, dv)
    tol = 2e-4 if dtype == "float32" else 4e-2
    assert float((got - ref).abs().max()) < tol


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(6, 2, 20, 12), (1, 1, 32, 32), (16, 2, 64, 32), (4, 4, 96, 96), (20, 2, 32, 48)],
                         ids=["odd", "one", "rep8", "d96", "rep10"])
@pytest.mark.parametrize("size,bs", [(10, 4), (64, 16), (1, 4), (96, 16), (300, 16)])
def test_attention_chunk_edges_pages_and_far_keys(device, dtype, shape, size, bs):
    H, G, dk, dv = shape
    _attention_case(device, dtype, H, G, dk, dv, size, bs, 260, 170)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(40, 2, 32, 16), (3, 1, 128, 128)], ids=["rep20", "d128"])
def test_attention_many_heads_per_key_head_and_large_heads(device, dtype, shape):
    """More query heads per key/value head than one wave's 16 slots; the largest matrix-core head size."""
    H, G, dk, dv = shape
    _attention_case(device, dtype, H, G, dk, dv, 96, 16, 150, 100)


@pytest.mark.parametrize("device,dtype", CASES)
def test_attention_without_sink_and_sink_alone(device, dtype):
    _attention_case(device, dtype, 4, 2, 32, 16, 16, 4, 70, 40, use_sink=False)
    # a huge sink takes all the weight: the output vanishes
    td = getattr(torch, dtype)
    sm = seq_meta(device, [(0, 0, 5)], 4, [[1, 0]])
    kc, vc = torch.zeros(8, 32, device=device, dtype=td), torch.zeros(8, 32, device=device, dtype=td)
    proj = torch.randn(5, 96).to(td).to(device)
    q = sq.qk_norm_cache(proj, 32, 32, 32, None, None, 0.0, sm, kc, vc)
    o = sq.masked_attention(q, kc, vc, 1, 1, 32, 32, sq.MASK_CHUNK, 3, 1.0, None, torch.full((1,), 80.0, device=device), 4, sm)
    assert float(o.float().abs().max()) < 1e-6


@pytest.mark.parametrize("device", OP_CASES)
def test_query_and_key_norms_span_all_heads(device):
    """The statistic is one per token over the whole projection, not one per head."""
    g = torch.Generator().manual_seed(1)
    nq, nk, nv = 24, 12, 10
    proj = torch.randn(6, nq + nk + nv + 3, generator=g)
    proj[:, :6] *= 20  # the first head is much larger than the others
    wq, wk = torch.randn(nq, generator=g), torch.randn(nk, generator=g)
    sm = seq_meta(device, [(0, 0, 6)], 4, [[2, 0]])
    kc, vc = torch.zeros(12, nk, device=device), torch.zeros(12, nv, device=device)
    q = sq.qk_norm_cache(proj.to(device), nq, nk, nv, wq.to(device), wk.to(device), 1e-5, sm, kc, vc)
    p64 = proj.to(F64)
    assert torch.allclose(q.cpu().to(F64), orc.unit_rms(p64[:, :nq], 1e-5) * wq.to(F64), atol=1e-5)
    rows = [8, 9, 10, 11, 0, 1]
    assert torch.allclose(kc.cpu()[rows].to(F64), orc.unit_rms(p64[:, nq:nq + nk], 1e-5) * wk.to(F64), atol=1e-5)
    assert torch.allclose(vc.cpu()[rows], proj[:, nq + nk:nq + nk + nv], atol=1e-6)


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("H,P,N,G,ng,taps", [(3, 12, 20, 3, 1, 2), (4, 16, 32, 2, 2, 4), (2, 40, 6, 1, 2, 3),
                                             (1, 64, 128, 1, 1, 4), (2, 8, 200, 2, 4, 1)])
def test_state_space_mixer_over_portions_and_slots(device, H, P, N, G, ng, taps):
    from xgserve.models.vizonex import SelectiveStateSpace
    W, eps = 40, 1e-5
    m = {"heads": H, "vdim": P, "state": N, "groups": G, "norm_groups": ng, "conv": taps}
    cfg = {"width": W, "vocab": 8, "canon": {"taps": 1}, "max_positions": 4,
           "layers": [{"type": "mamba2", "mixer": m, "mlp": None}]}
    Wt = orc.random_weights(cfg, seed=N)
    g = torch.Generator().manual_seed(3)
    lens = [90, 6, 1]
    hs = [torch.randn(n, W, generator=g) for n in lens]
    refs = [orc.ssm_mixer(Wt, "l0.mix.", m, h.to(F64), eps) for h in hs]
    mix = SelectiveStateSpace(W, m, eps, device, torch.float32)
    for dst, n in ((mix.in_proj, "in"), (mix.conv_w, "conv"), (mix.conv_b, "conv.b"), (mix.dt_bias, "dt_bias"),
                   (mix.A_log, "A_log"), (mix.D, "D"), (mix.norm, "norm"), (mix.o, "o")):
        dst.data.copy_(Wt["l0.mix." + n].float())
    lc = LayerCache(mix_conv=torch.full((4, taps - 1, mix.ch), 30.0, device=device),
                    ssm=torch.full((4, H, N, P), 50.0, device=device))  # stale state of earlier owners
    got = in_portions(device, hs, [[2, 1, 40, 1, 1, 45], [3, 1, 2], [1]], [1, 3, 0], lambda x, sm: mix(x, sm, lc, 4))
    for i in range(3):
        assert torch.allclose(got[i], refs[i], atol=3e-4, rtol=1e-3), i
    # the carried state equals the oracle's final state
    st = []
    orc.ssm_mixer(Wt, "l0.mix.", m, hs[0].to(F64), eps, st)
    assert torch.allclose(lc.ssm[1].cpu().to(F64), torch.stack(st), atol=3e-4, rtol=1e-3)


@pytest.mark.parametrize("device", OP_CASES)
def test_group_norm_of_the_gated_output(device):
    g = torch.Generator().manual_seed(2)
    y, z, w = torch.randn(5, 48, generator=g), torch.randn(5, 60, generator=g), torch.randn(48, generator=g)
    for ng in (1, 3, 48):
        v = (y.to(F64) * orc.silu(z[:, 7:55].to(F64))).reshape(5, ng, 48 // ng)
        ref = orc.unit_rms(v, 1e-5).reshape(5, 48) * w.to(F64)
        got = sq.gated_group_norm(y.to(device), z.to(device)[:, 7:55], w.to(device), 1e-5, ng, torch.float32)
        assert torch.allclose(got.cpu().to(F64), ref, atol=1e-5), ng


@pytest.mark.parametrize("device", OP_CASES)
def test_gated_activations_and_their_clamps(device):
    g = torch.linspace(-8, 8, 801).reshape(1, -1)
    u = torch.linspace(5, -5, 801).reshape(1, -1)
    x = torch.cat([g, u], 1)
    got = sq.glu_act(x.to(device), sq.GLU_GELU_TANH).cpu().to(F64)
    assert torch.allclose(got, orc.gelu_tanh(g.to(F64)) * u.to(F64), atol=1e-5)
    lim = 1.5
    gc, uc = g.to(F64).clamp(max=lim), u.to(F64).clamp(-lim, lim)
    got = sq.glu_act(x.to(device), sq.GLU_CLAMPED, lim, 1.702).cpu().to(F64)
    assert torch.allclose(got, gc * torch.sigmoid(1.702 * gc) * (uc + 1.0), atol=1e-5)


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("E,count,keep,top", [(16, 4, 3, 2), (6, 3, 2, 3), (5, 5, 2, 2), (4, 1, 1, 1), (72, 8, 3, 6),
                                              (160, 4, 1, 8)])
def test_router_groups_correction_and_weights(device, E, count, keep, top):
    """Strongly negative corrections make every selection score negative, so an expert outside the eligible
    groups has to be excluded outright (scoring it 0 would let it win). The weights are the plain scores times
    the scale."""
    g = torch.Generator().manual_seed(E)
    z = torch.randn(40, E, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.5 - 3.0
    r = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": count, "keep": keep}}
    ref = orc.route_scores(z.to(F64), corr.to(F64), r)
    ids, wts = sq.grouped_router(z.to(device), corr.to(device), count, keep, top, 1.7)
    for t in range(40):
        got = sorted(zip(ids[t].tolist(), wts[t].tolist()))
        want = sorted(ref[t])
        assert [e for e, _ in got] == [e for e, _ in want], t
        assert all(abs(a - b) < 1e-5 for (_, a), (_, b) in zip(got, want)), t


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("W,ff,E,top,T", [(40, 24, 6, 3, 50), (64, 32, 16, 2, 300), (96, 80, 3, 1, 7), (64, 16, 40, 4, 1),
                                          (64, 48, 4, 2, 200), (128, 64, 2, 2, 333)])
def test_experts_weighted_sum(device, dtype, W, ff, E, top, T):
    from xgserve.models.vizonex import GroupedRouterMoE
    td = getattr(torch, dtype)
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": 1.2}, "shared": {"ff": 2 * ff, "limit": 0.8},
           "router": {"experts": E, "top": top, "scale": 1.3, "groups": {"count": 1, "keep": 1}}}
    cfg = {"width": W, "vocab": 8, "canon": {"taps": 1}, "max_positions": 4,
           "layers": [{"type": "attention", "mixer": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8}, "mlp": mlp}]}
    Wt = orc.random_weights(cfg, seed=E)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(T, W, generator=g).to(td)
    ref = orc.moe_ff(Wt, "l0.mlp.", mlp, h.to(F64))
    mod = GroupedRouterMoE(W, mlp, device, td)
    mod.router.data.copy_(Wt["l0.mlp.router"].float())
    mod.correction.data.copy_(Wt["l0.mlp.correction"].float())
    for e in range(E):
        mod.w13.data[e, :ff] = Wt[f"l0.mlp.e{e}.gate"].to(td)
        mod.w13.data[e, ff:] = Wt[f"l0.mlp.e{e}.up"].to(td)
        mod.w2.data[e] = Wt[f"l0.mlp.e{e}.down"].to(td)
    mod.shared.gate_up.data[:2 * ff] = Wt["l0.mlp.shared.gate"].to(td)
    mod.shared.gate_up.data[2 * ff:] = Wt["l0.mlp.shared.up"].to(td)
    mod.shared.down.data.copy_(Wt["l0.mlp.shared.down"].to(td))
    shared, routed = mod(h.float().to(device), h.to(device))
    got = (shared.float() + routed).cpu().to(F64)
    tol = 2e-4 if dtype == "float32" else 5e-2
    assert float((got - ref).abs().max()) < tol * max(1.0, float(ref.abs().max()))
