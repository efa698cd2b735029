"""Dofivik: a decoder made of a configured list of layers on the paged / slotted engine.

Every layer is  x <- norm1(alpha x + mixer(h1)),  then (if it has a feed-forward)
x <- norm2(alpha x + ff(h2)),  where each sublayer reads h = x + conv(x), a short causal
depthwise convolution over time, and the norms are RMS norms with a weight stored around
zero (applied as 1 + w). The residual stream x is fp32 throughout.

Mixers:
  * "latent_attention": queries through a normed low-rank latent; keys and values are
    up-projections of ONE normed latent per token plus ONE rotary key shared by all heads,
    so the paged cache holds only [latent | rotated key] per token. Attention runs in latent
    space (the key up-projection is folded into the query, the value up-projection follows
    the softmax), over a sliding window, with a per-head sigmoid output gate. A layer with
    "kv_from" reads another layer's cache rows with its own up-projections.
  * "general_delta": a generalized delta rule with per-channel decay and removal rate on a
    [dim x dim] fp32 state per head, carried per sequence slot.
Feed-forward: dense, xIELU activation, biases.

What a sequence carries between steps (ModelRunner allocates it through alloc_cache):
pages of latent rows (attention layers that own a cache), and per state slot the last
taps - 1 inputs of every convolution and the delta-rule states.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops import seqmix as sq
from ..parallel.state import get_state
from .base import AttnMeta
from .config import ModelConfig
from .seq_cache import LayerCache, SeqCache


def _p(t):
    return nn.Parameter(t, requires_grad=False)


def _softplus(v: float) -> float:
    return v if v > 30 else math.log1p(math.exp(v))


class LatentAttentionMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.dn, self.rd, self.dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
        self.R, self.Rq = m["kv_rank"], m["q_rank"]
        self.window, self.scale = int(m["mask"]["size"]), float(m["scale"])
        self.rot_dims, self.rot_base = int(m["rot"]["dims"]), float(m["rot"]["base"])
        if self.rot_dims % 2 or self.rot_dims > self.rd:
            raise ValueError("rot.dims must be even and at most rot_dim")
        self.kv_from = m.get("kv_from")
        self.own_kv = self.kv_from is None
        self.eps = eps
        # fused input projection rows: [query latent | (kv latent | shared rotary key) | head gates]
        self.off_kv = self.Rq if self.own_kv else -1
        self.off_g = self.Rq + (self.R + self.rd if self.own_kv else 0)
        self.in_proj = _p(e(self.off_g + self.H, width))
        self.q_norm = _p(f(self.Rq))
        self.kv_norm = _p(f(self.R)) if self.own_kv else None
        self.uq = _p(e(self.H * (self.dn + self.rd), self.Rq))
        self.uk = _p(e(self.H * self.dn, self.R))
        self.uv = _p(e(self.H * self.dv, self.R))
        self.o = _p(e(width, self.H * self.dv))

    def forward(self, h, sm: sq.SeqMeta, cache_rows, rot, block_size):
        T, H, dq = h.shape[0], self.H, self.dn + self.rd
        proj = F.linear(h, self.in_proj)
        cq = sq.latent_prep(proj, 0, self.Rq, self.off_kv, self.R, self.rd, self.q_norm, self.kv_norm, self.eps, rot,
                            self.rot_dims, sm, cache_rows)
        q = F.linear(cq, self.uq).view(T, H, dq)
        qabs = torch.bmm(q[:, :, :self.dn].transpose(0, 1), self.uk.view(H, self.dn, self.R))  # [H, T, R]
        o_lat = sq.latent_attention(qabs, q, self.dn, proj[:, self.off_g:], cache_rows, rot, self.rot_dims, self.window,
                                    self.scale, block_size, sm)
        o = torch.bmm(o_lat, self.uv.view(H, self.dv, self.R).transpose(1, 2))  # [H, T, dv]
        return F.linear(sq.heads_to_rows(o), self.o)


class DeltaRuleMixer(nn.Module):
    def __init__(self, width: int, m: dict, lowrank: int, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.D = m["heads"], m["dim"]
        self.HD, self.lr, self.eps = self.H * self.D, lowrank, eps
        # fused input projection rows: [r | k | v | gate | removal logits | decay low-rank]
        self.in_proj = _p(e(5 * self.HD + lowrank, width))
        self.w2 = _p(e(self.HD, lowrank))
        self.w0, self.a_bias, self.norm = _p(f(self.HD)), _p(f(self.HD)), _p(f(self.HD))
        self.o = _p(e(width, self.HD))

    def forward(self, h, sm: sq.SeqMeta, state):
        HD = self.HD
        proj = F.linear(h, self.in_proj)
        wl = F.linear(sq.tanh_cols(proj, 5 * HD, self.lr), self.w2)
        o = sq.delta_rule_scan(proj, 0, HD, 2 * HD, 4 * HD, wl, self.a_bias, self.w0, state, self.H, self.D, sm)
        y = sq.delta_rule_out(o, self.norm, proj[:, 3 * HD:4 * HD], self.eps, self.H, self.D, h.dtype)
        return F.linear(y, self.o)


class XieluMLP(nn.Module):
    def __init__(self, width: int, ff: int, device, dtype):
        super().__init__()
        self.up = _p(torch.empty(ff, width, device=device, dtype=dtype))
        self.down = _p(torch.empty(width, ff, device=device, dtype=dtype))
        self.up_b = _p(torch.zeros(ff, device=device, dtype=torch.float32))
        self.down_b = _p(torch.zeros(width, device=device, dtype=torch.float32))
        self.act = _p(torch.zeros(2, device=device, dtype=torch.float32))
        self.sp, self.cn = _softplus(0.0), 0.5 + _softplus(0.0)

    def set_act(self):
        p, q = (float(v) for v in self.act.detach().cpu())
        self.sp, self.cn = _softplus(p), 0.5 + _softplus(q)

    def forward(self, h):
        """W_down act(W_up h + b_up); the down bias is added by the caller's norm."""
        return F.linear(sq.xielu(F.linear(h, self.up), self.up_b, self.sp, self.cn), self.down)


class DofivikLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, lowrank: int, device, dtype):
        super().__init__()
        W, taps = cfg.hidden_size, cfg.canon_taps
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.kind = spec["type"]
        self.alpha, self.eps = cfg.postln_alpha, cfg.norm_eps
        if self.kind == "latent_attention":
            self.mix = LatentAttentionMixer(W, spec["mixer"], cfg.norm_eps, device, dtype)
        else:
            self.mix = DeltaRuleMixer(W, spec["mixer"], lowrank, cfg.norm_eps, device, dtype)
        self.norm1, self.canon1 = _p(f(W)), _p(f(W, taps))
        self.mlp = None
        if spec.get("mlp") is not None:
            self.mlp = XieluMLP(W, spec["mlp"]["ff"], device, dtype)
            self.norm2, self.canon2 = _p(f(W)), _p(f(W, taps))

    def forward(self, x, sm: sq.SeqMeta, lc: LayerCache, rot, block_size, dtype):
        h = sq.causal_conv_residual(x, self.canon1, lc.conv1, sm, dtype)
        if self.kind == "latent_attention":
            y = self.mix(h, sm, lc.latent, rot, block_size)
        else:
            y = self.mix(h, sm, lc.delta)
        sq.scaled_add_rmsnorm(x, y, self.norm1, self.eps, self.alpha, None, 1.0)
        if self.mlp is not None:
            h = sq.causal_conv_residual(x, self.canon2, lc.conv2, sm, dtype)
            sq.scaled_add_rmsnorm(x, self.mlp(h), self.norm2, self.eps, self.alpha, self.mlp.down_b, 1.0)
        return x


def _lowrank_of(spec: dict, default: int = 32) -> int:
    return int(spec["mixer"].get("decay_rank", default))


class DofivikForCausalLM(nn.Module):
    has_sequence_state = True   # recurrent / convolution state per slot: no prefix reuse, no draft verification

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp: Optional[int] = None,
                 rank: Optional[int] = None, decay_ranks: Optional[Dict[int, int]] = None):
        super().__init__()
        tp = get_state().tp_size if tp is None else tp
        if tp != 1:
            raise ValueError("Dofivik runs with tp=1 (use DP replicas to scale)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Dofivik runs in bfloat16 or float32")
        self.cfg, self.tp, self.rank = cfg, 1, 0
        self.device, self.dtype = torch.device(device), dtype
        W = cfg.hidden_size
        self.embed = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.layers = nn.ModuleList([
            DofivikLayer(cfg, spec, (decay_ranks or {}).get(i, _lowrank_of(spec)), device, dtype)
            for i, spec in enumerate(cfg.layer_specs)])
        self.final_norm = _p(torch.zeros(W, device=device, dtype=torch.float32))
        self.head = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.num_kv_heads_local = 1
        self._rot: Dict[tuple, torch.Tensor] = {}
        self._rot_len = 0
        self.set_max_positions(min(cfg.max_position, 4096))

    # ------------------------------------------------------------------ positions
    def set_max_positions(self, n: int) -> None:
        """(Re)build the rotation tables for positions [0, n) -- the runner passes its max_model_len."""
        if n <= self._rot_len:
            return
        self._rot = {}
        for L in self.layers:
            if L.kind == "latent_attention":
                key = (L.mix.rot_dims, L.mix.rot_base)
                if key not in self._rot:
                    self._rot[key] = sq.build_rot_table(key[0], key[1], n, self.device)
        self._rot_len = n

    # ------------------------------------------------------------------ cache / state
    def alloc_cache(self, num_blocks: int, block_size: int, max_num_seqs: int) -> SeqCache:
        dev, W, nh = self.device, self.cfg.hidden_size, self.cfg.canon_taps - 1
        sc = SeqCache(block_size=block_size)
        for L in self.layers:
            lc = LayerCache(conv1=torch.zeros(max_num_seqs, nh, W, dtype=torch.float32, device=dev))
            if L.mlp is not None:
                lc.conv2 = torch.zeros(max_num_seqs, nh, W, dtype=torch.float32, device=dev)
            if L.kind == "latent_attention":
                if L.mix.own_kv:
                    lc.latent = torch.zeros(num_blocks * block_size, L.mix.R + L.mix.rd, dtype=self.dtype, device=dev)
                else:
                    lc.latent = sc.layers[L.mix.kv_from].latent
            else:
                lc.delta = torch.zeros(max_num_seqs, L.mix.H, L.mix.D, L.mix.D, dtype=torch.float32, device=dev)
            sc.layers.append(lc)
        return sc

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = torch.tensor([], dtype=self.dtype).element_size()
        return block_size * sum((L.mix.R + L.mix.rd) * esz for L in self.layers
                                if L.kind == "latent_attention" and L.mix.own_kv)

    def state_bytes_per_slot(self) -> int:
        W, nh = self.cfg.hidden_size, self.cfg.canon_taps - 1
        n = 0
        for L in self.layers:
            n += nh * W * (2 if L.mlp is not None else 1)
            if L.kind == "general_delta":
                n += L.mix.H * L.mix.D * L.mix.D
        return 4 * n

    # ------------------------------------------------------------------ weights
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        g = torch.Generator().manual_seed(seed)

        def mat(p):
            p.copy_((torch.randn(p.shape, generator=g) / math.sqrt(p.shape[1])).to(p.dtype))

        def vec(p, std, mean=0.0):
            p.copy_(torch.randn(p.shape, generator=g) * std + mean)
        self.embed.copy_(torch.randn(self.embed.shape, generator=g).to(self.dtype))
        mat(self.head)
        vec(self.final_norm, 0.1)
        for L in self.layers:
            vec(L.norm1, 0.1)
            vec(L.canon1, 0.3)
            m = L.mix
            if L.kind == "latent_attention":
                for p in (m.in_proj, m.uq, m.uk, m.uv, m.o):
                    mat(p)
                vec(m.q_norm, 0.1, 1.0)
                if m.own_kv:
                    vec(m.kv_norm, 0.1, 1.0)
            else:
                for p in (m.in_proj, m.w2, m.o):
                    mat(p)
                vec(m.w0, 1.0)
                vec(m.a_bias, 0.5)
                vec(m.norm, 0.1, 1.0)
            if L.mlp is not None:
                vec(L.norm2, 0.1)
                vec(L.canon2, 0.3)
                mat(L.mlp.up)
                mat(L.mlp.down)
                vec(L.mlp.up_b, 0.1)
                vec(L.mlp.down_b, 0.1)
                vec(L.mlp.act, 0.5)
        self.finalize_weights()

    def finalize_weights(self):
        """Host-side constants derived from loaded weights (activation shape numbers)."""
        for L in self.layers:
            if L.mlp is not None:
                L.mlp.set_act()

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, cache: SeqCache):
        sm = meta.seq
        if sm is None:
            raise ValueError("Dofivik needs the step's per-sequence metadata (AttnMeta.seq)")
        x = sq.embed_rows(input_ids, self.embed)
        for L, lc in zip(self.layers, cache.layers):
            rot = self._rot[(L.mix.rot_dims, L.mix.rot_base)] if L.kind == "latent_attention" else None
            x = L(x, sm, lc, rot, cache.block_size, self.dtype)
        self.last_hidden = x
        return sq.scaled_add_rmsnorm(x, None, self.final_norm, self.cfg.norm_eps, 1.0, None, 1.0, inplace=False,
                                     out_dtype=self.dtype)

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head)

    def set_moe_comm(self, mode: str):
        pass


def count_params(cfg: ModelConfig) -> int:
    W, V, taps = cfg.hidden_size, cfg.vocab_size, cfg.canon_taps
    n = 2 * V * W + W
    for spec in cfg.layer_specs:
        m = spec["mixer"]
        n += W + W * taps
        if spec["type"] == "latent_attention":
            H, dn, rd, dv, R, Rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            n += Rq * W + Rq + H * (dn + rd) * Rq + H * dn * R + H * dv * R + H * W + W * H * dv
            if "kv_from" not in m:
                n += (R + rd) * W + R
        else:
            HD, lr = m["heads"] * m["dim"], _lowrank_of(spec)
            n += 5 * HD * W + lr * W + HD * lr + 3 * HD + W * HD
        if spec.get("mlp") is not None:
            ff = spec["mlp"]["ff"]
            n += W + W * taps + 2 * W * ff + ff + W + 2
    return n
