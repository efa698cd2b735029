"""Vizonex: a decoder made of a configured list of parallel blocks on the paged / slotted engine.

    x_0 = embed[token] + pos[position]                       (learned position vectors)
    n   = rmsnorm(x) * g                                     (ONE norm per block)
    x  <- x + a1 * mixer(n + conv(n)) + a2 * ff(n)           (both sublayers read the same norm;
                                                              a1 / a2 per-channel layer scales)

`conv` is a short causal depthwise convolution over time (no bias); only the mixer reads through
it. The residual stream x is fp32 throughout; the residual sum of a block and the norm of the next
one run in one kernel.

Mixers (reusable modules, every constant a parameter):
  * `ChunkedSinkAttention` ("attention"): grouped-query attention without positional rotation;
    queries and keys are RMS-normed over their WHOLE projection (all heads at once); per-head
    temperature; a query sees the keys of its own chunk of `mask.size` positions only (chunks
    counted from the sequence's start); the softmax denominator holds one extra learned term per
    head (a sink: no key, no value).
  * `SelectiveStateSpace` ("mamba2"): input projection [z | x | B | C | dt], a short convolution +
    silu over [x | B | C], a scalar-decay state-space recurrence on an fp32 [state x vdim] state per
    head and slot, gating by silu(z) followed by a group RMS norm, output projection.
Feed-forward: `GatedMLP` (gelu-tanh gate) or `GroupedRouterMoE` (sigmoid router with a selection-only
correction and group-limited top-k over clamped-GLU experts, plus an always-on shared expert).

What a sequence carries between steps (ModelRunner allocates it through alloc_cache): K / V pages
of the attention layers; per state slot the last taps - 1 inputs of every block's input convolution,
the last taps - 1 inputs of every state-space layer's own convolution, and its recurrent state.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops import seqmix as sq
from ..parallel.state import get_state
from .base import AttnMeta
from .config import ModelConfig
from .seq_cache import LayerCache, SeqCache

GLU_ALPHA = 1.702  # slope of the sigmoid in the clamped GLU of the experts


def _p(t):
    return nn.Parameter(t, requires_grad=False)


class ChunkedSinkAttention(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        self.size, self.scale, self.eps = int(m["mask"]["size"]), float(m["scale"]), eps
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        self.qkv = _p(e(self.nq + self.nk + self.nv, width))   # fused rows [q | k | v]
        self.q_norm, self.k_norm = _p(f(self.nq)), _p(f(self.nk))
        self.temp, self.sink = _p(f(self.H)), _p(f(self.H))
        self.o = _p(e(width, self.H * self.dv))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int):
        proj = F.linear(h, self.qkv)
        q = sq.qk_norm_cache(proj, self.nq, self.nk, self.nv, self.q_norm, self.k_norm, self.eps, sm, lc.k, lc.v)
        o = sq.masked_attention(q, lc.k, lc.v, self.H, self.G, self.dk, self.dv, sq.MASK_CHUNK, self.size, self.scale,
                                self.temp, self.sink, block_size, sm)
        return F.linear(o, self.o)


class SelectiveStateSpace(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.P, self.N, self.G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
        self.ng, self.taps, self.eps = int(m["norm_groups"]), int(m["conv"]), eps
        self.inner = self.H * self.P
        self.ch = self.inner + 2 * self.G * self.N            # channels of the short convolution: [x | B | C]
        self.in_proj = _p(e(2 * self.inner + 2 * self.G * self.N + self.H, width))  # rows [z | x | B | C | dt]
        self.conv_w, self.conv_b = _p(f(self.ch, self.taps)), _p(f(self.ch))
        self.dt_bias, self.A_log, self.D = _p(f(self.H)), _p(f(self.H)), _p(f(self.H))
        self.norm = _p(f(self.inner))
        self.o = _p(e(width, self.inner))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int):
        inner, ch = self.inner, self.ch
        proj = F.linear(h, self.in_proj)
        xbc = sq.causal_conv(proj[:, inner:inner + ch], self.conv_w, self.conv_b, lc.mix_conv, sm, h.dtype, residual=False,
                             silu=True)
        y = sq.ssm_scan(xbc, proj[:, inner + ch:], self.dt_bias, self.A_log, self.D, lc.ssm, self.H, self.G, self.N,
                        self.P, sm)
        return F.linear(sq.gated_group_norm(y, proj[:, :inner], self.norm, self.eps, self.ng, h.dtype), self.o)


class GatedMLP(nn.Module):
    """W_down (act(W_gate h) * up(W_up h)) with a gated activation of ops.seqmix.glu_act."""

    def __init__(self, width: int, ff: int, kind: int, limit: float, device, dtype):
        super().__init__()
        self.ff, self.kind, self.limit = int(ff), kind, float(limit)
        self.gate_up = _p(torch.empty(2 * self.ff, width, device=device, dtype=dtype))   # rows [gate | up]
        self.down = _p(torch.empty(width, self.ff, device=device, dtype=dtype))

    def forward(self, h):
        return F.linear(sq.glu_act(F.linear(h, self.gate_up), self.kind, self.limit, GLU_ALPHA), self.down)


class GroupedRouterMoE(nn.Module):
    def __init__(self, width: int, mlp: dict, device, dtype):
        super().__init__()
        r = mlp["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        self.count, self.keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
        self.rscale = float(r["scale"])
        self.ff, self.limit = int(mlp["expert"]["ff"]), float(mlp["expert"]["limit"])
        self.router = _p(torch.zeros(self.E, width, device=device, dtype=torch.float32))
        self.correction = _p(torch.zeros(self.E, device=device, dtype=torch.float32))
        self.w13 = _p(torch.empty(self.E, 2 * self.ff, width, device=device, dtype=dtype))  # per expert rows [gate | up]
        self.w2 = _p(torch.empty(self.E, width, self.ff, device=device, dtype=dtype))
        sh = mlp.get("shared")
        self.shared = GatedMLP(width, sh["ff"], sq.GLU_CLAMPED, sh["limit"], device, dtype) if sh is not None else None

    def forward(self, n32, nact):
        """(shared expert's output as an activation tensor or None, routed sum fp32)."""
        ids, wts = sq.grouped_router(F.linear(n32, self.router), self.correction, self.count, self.keep, self.top,
                                     self.rscale)
        routed = sq.routed_experts(nact, self.w13, self.w2, ids, wts, sq.GLU_CLAMPED, self.limit, GLU_ALPHA)
        return (self.shared(nact) if self.shared is not None else None), routed


class VizonexLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, device, dtype):
        super().__init__()
        W, taps = cfg.hidden_size, cfg.canon_taps
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.kind, self.eps = spec["type"], cfg.norm_eps
        if self.kind == "attention":
            self.mix = ChunkedSinkAttention(W, spec["mixer"], cfg.norm_eps, device, dtype)
        else:
            self.mix = SelectiveStateSpace(W, spec["mixer"], cfg.norm_eps, device, dtype)
        self.norm1, self.ls1, self.canon1 = _p(f(W)), _p(f(W)), _p(f(W, taps))
        mlp = spec.get("mlp")
        self.mlp, self.moe, self.ls2 = None, False, None
        if mlp is not None:
            self.ls2 = _p(f(W))
            self.moe = mlp["kind"] == "moe"
            self.mlp = GroupedRouterMoE(W, mlp, device, dtype) if self.moe else \
                GatedMLP(W, mlp["ff"], sq.GLU_GELU_TANH, 0.0, device, dtype)

    def forward(self, x, n32, nact, sm: sq.SeqMeta, lc: LayerCache, block_size: int, next_norm, want_f32: bool):
        """x: fp32 residual (updated in place); n32 / nact: this block's norm of x. Returns (x, the next
        norm of x as fp32 or None, and as an activation tensor)."""
        h = sq.causal_conv(n32, self.canon1, None, lc.conv1, sm, nact.dtype, residual=True)
        y1 = self.mix(h, sm, lc, block_size)
        y2 = y3 = None
        if self.mlp is not None:
            if self.moe:
                y2, y3 = self.mlp(n32, nact)
            else:
                y2 = self.mlp(nact)
        n32, nact = sq.residual_norm(x, y1, self.ls1, y2, y3, self.ls2, next_norm, self.eps, nact.dtype, want_f32)
        return x, n32, nact


class VizonexForCausalLM(nn.Module):
    has_sequence_state = True   # recurrent / convolution state per slot: no prefix reuse, no draft verification

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp: Optional[int] = None,
                 rank: Optional[int] = None):
        super().__init__()
        tp = get_state().tp_size if tp is None else tp
        if tp != 1:
            raise ValueError("Vizonex runs with tp=1 (use DP replicas to scale)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Vizonex runs in bfloat16 or float32")
        self.cfg, self.tp, self.rank = cfg, 1, 0
        self.device, self.dtype = torch.device(device), dtype
        W = cfg.hidden_size
        self.embed = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.pos = _p(torch.empty(cfg.max_position, W, device=device, dtype=dtype))
        self.layers = nn.ModuleList([VizonexLayer(cfg, spec, device, dtype) for spec in cfg.layer_specs])
        self.final_norm = _p(torch.zeros(W, device=device, dtype=torch.float32))
        self.head = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.num_kv_heads_local = 1

    # ------------------------------------------------------------------ cache / state
    def alloc_cache(self, num_blocks: int, block_size: int, max_num_seqs: int) -> SeqCache:
        dev, W, nh = self.device, self.cfg.hidden_size, self.cfg.canon_taps - 1
        f32 = dict(dtype=torch.float32, device=dev)
        sc = SeqCache(block_size=block_size)
        rows = num_blocks * block_size
        for L in self.layers:
            lc, m = LayerCache(conv1=torch.zeros(max_num_seqs, nh, W, **f32)), L.mix
            if L.kind == "attention":
                lc.k = torch.zeros(rows, m.nk, dtype=self.dtype, device=dev)
                lc.v = torch.zeros(rows, m.nv, dtype=self.dtype, device=dev)
            else:
                lc.mix_conv = torch.zeros(max_num_seqs, m.taps - 1, m.ch, **f32)
                lc.ssm = torch.zeros(max_num_seqs, m.H, m.N, m.P, **f32)
            sc.layers.append(lc)
        return sc

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = torch.tensor([], dtype=self.dtype).element_size()
        return block_size * sum((L.mix.nk + L.mix.nv) * esz for L in self.layers if L.kind == "attention")

    def state_bytes_per_slot(self) -> int:
        n = 0
        for L in self.layers:
            n += (self.cfg.canon_taps - 1) * self.cfg.hidden_size
            if L.kind != "attention":
                n += (L.mix.taps - 1) * L.mix.ch + L.mix.H * L.mix.N * L.mix.P
        return 4 * n

    # ------------------------------------------------------------------ weights
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        g = torch.Generator().manual_seed(seed)

        def mat(p, gain=1.0):
            p.copy_((torch.randn(p.shape, generator=g) * gain / math.sqrt(p.shape[-1])).to(p.dtype))

        def vec(p, std, mean=0.0):
            p.copy_(torch.randn(p.shape, generator=g) * std + mean)
        self.embed.copy_(torch.randn(self.embed.shape, generator=g).to(self.dtype))
        self.pos.copy_((torch.randn(self.pos.shape, generator=g) * 0.3).to(self.dtype))
        mat(self.head)
        vec(self.final_norm, 0.1, 1.0)
        for L in self.layers:
            vec(L.norm1, 0.1, 1.0)
            vec(L.ls1, 0.1, 0.5)
            vec(L.canon1, 0.3)
            m = L.mix
            if L.kind == "attention":
                mat(m.qkv)
                mat(m.o)
                vec(m.q_norm, 0.1, 1.0)
                vec(m.k_norm, 0.1, 1.0)
                vec(m.temp, 0.1, 1.0)
                vec(m.sink, 0.5)
            else:
                mat(m.in_proj)
                mat(m.o)
                vec(m.conv_w, 0.4)
                vec(m.conv_b, 0.1)
                vec(m.dt_bias, 0.5, -1.0)
                vec(m.A_log, 0.5, -0.5)
                vec(m.D, 0.3, 1.0)
                vec(m.norm, 0.1, 1.0)
            if L.mlp is None:
                continue
            vec(L.ls2, 0.1, 0.5)
            if L.moe:
                mat(L.mlp.router, 2.0)
                vec(L.mlp.correction, 0.2)
                mat(L.mlp.w13)
                mat(L.mlp.w2)
                if L.mlp.shared is not None:
                    mat(L.mlp.shared.gate_up)
                    mat(L.mlp.shared.down)
            else:
                mat(L.mlp.gate_up)
                mat(L.mlp.down)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, cache: SeqCache):
        sm = meta.seq
        if sm is None:
            raise ValueError("Vizonex needs the step's per-sequence metadata (AttnMeta.seq)")
        x = sq.embed_rows(input_ids, self.embed, self.pos, sm.positions)
        n32, nact = sq.residual_norm(x, None, None, None, None, None, self.layers[0].norm1, self.cfg.norm_eps,
                                     self.dtype, True)
        last = len(self.layers) - 1
        for i, (L, lc) in enumerate(zip(self.layers, cache.layers)):
            nxt = self.layers[i + 1].norm1 if i < last else self.final_norm
            x, n32, nact = L(x, n32, nact, sm, lc, cache.block_size, nxt, i < last)
        self.last_hidden = x
        return nact

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head)

    def set_moe_comm(self, mode: str):
        pass


def count_params(cfg: ModelConfig) -> int:
    W, V, taps = cfg.hidden_size, cfg.vocab_size, cfg.canon_taps
    n = 2 * V * W + W + cfg.max_position * W
    for spec in cfg.layer_specs:
        m = spec["mixer"]
        n += 2 * W + W * taps
        if spec["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            n += (H * dk + G * dk + G * dv) * W + H * dk + G * dk + 2 * H + W * H * dv
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = H * P + 2 * G * N
            n += (2 * H * P + 2 * G * N + H) * W + ch * (m["conv"] + 1) + 3 * H + H * P + W * H * P
        mlp = spec.get("mlp")
        if mlp is None:
            continue
        n += W
        if mlp["kind"] == "dense":
            n += 3 * W * mlp["ff"]
        else:
            E = mlp["router"]["experts"]
            n += E * 3 * W * mlp["expert"]["ff"] + E * W + E
            if mlp.get("shared") is not None:
                n += 3 * W * mlp["shared"]["ff"]
    return n
