"""Slow, dense, fp64 oracle of the Dofivik design: one function per mechanism, whole sequences,
no cache, no batching. It shares nothing with xgserve's model or ops; the tests compare the
framework against it. Weights are a dict of checkpoint tensor names -> fp64 tensors.

Notation: x_t is the residual row of token t (t = 0 is the sequence's first token).
"""
import math

import torch

F64 = torch.float64


def unit_rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def shifted_conv(h, w):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j); rows before t = 0 are zero. h [T, C], w [C, taps]."""
    T, C = h.shape
    taps = w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def rotate_interleaved(v, positions, dims, base):
    """Pairs (2i, 2i+1), i < dims/2, of the last axis turn by angle p * base^(-2i/dims); the rest stays."""
    out = v.clone()
    for n, p in enumerate(positions):
        for i in range(dims // 2):
            ang = float(p) * base ** (-2.0 * i / dims)
            c, s = math.cos(ang), math.sin(ang)
            a, b = v[n, ..., 2 * i].clone(), v[n, ..., 2 * i + 1].clone()
            out[n, ..., 2 * i] = a * c - b * s
            out[n, ..., 2 * i + 1] = b * c + a * s
    return out


def latent_kv(Wt, pre, m, h, eps):
    """The cached quantities of a latent-attention layer: normed latent [T, R] and rotated shared key [T, rd]."""
    R = m["kv_rank"]
    z = h @ Wt[pre + "dkv"].T
    lat = unit_rms(z[:, :R], eps) * Wt[pre + "dkv.norm"]
    key = rotate_interleaved(z[:, R:], range(h.shape[0]), m["rot"]["dims"], m["rot"]["base"])
    return lat, key


def latent_attention(Wt, pre, m, h, lat, key, eps):
    """Per-head keys / values are up-projections of the latent; the rotary key part is shared by all heads."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    qlat = unit_rms(h @ Wt[pre + "dq"].T, eps) * Wt[pre + "dq.norm"]
    q = (qlat @ Wt[pre + "uq"].T).reshape(T, H, dn + dr)
    q_plain = q[:, :, :dn]
    q_rot = rotate_interleaved(q[:, :, dn:], range(T), m["rot"]["dims"], m["rot"]["base"])
    k_plain = (lat @ Wt[pre + "uk"].T).reshape(T, H, dn)
    val = (lat @ Wt[pre + "uv"].T).reshape(T, H, dv)
    gate = torch.sigmoid(h @ Wt[pre + "g"].T)
    win = m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = max(0, i - win + 1)
        for hd in range(H):
            sc = torch.stack([(q_plain[i, hd] @ k_plain[j, hd] + q_rot[i, hd] @ key[j]) * m["scale"]
                              for j in range(lo, i + 1)])
            p = torch.softmax(sc, 0)
            out[i, hd] = (p[:, None] * val[lo:i + 1, hd]).sum(0) * gate[i, hd]
    return out.reshape(T, H * dv) @ Wt[pre + "o"].T


def delta_rule(Wt, pre, m, h, eps):
    """S <- diag(w) S - (a*u)(u^T S) + k v^T with both terms reading the old S; o = S^T r."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ Wt[pre + "r"].T).reshape(T, H, D)
    k = (h @ Wt[pre + "k"].T).reshape(T, H, D)
    v = (h @ Wt[pre + "v"].T).reshape(T, H, D)
    lg = torch.tanh(h @ Wt[pre + "w1"].T) @ Wt[pre + "w2"].T + Wt[pre + "w0"]
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(lg)).reshape(T, H, D)
    a = torch.sigmoid(h @ Wt[pre + "a"].T + Wt[pre + "a.b"]).reshape(T, H, D)
    out = torch.zeros(T, H, D, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, D, dtype=F64)
        for t in range(T):
            u = k[t, hd] / torch.sqrt((k[t, hd] ** 2).sum() + 1e-6)
            old = S
            S = w[t, hd][:, None] * old - torch.outer(a[t, hd] * u, u @ old) + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ r[t, hd]
    y = unit_rms(out, eps).reshape(T, H * D) * Wt[pre + "norm"] * torch.sigmoid(h @ Wt[pre + "g"].T)
    return y @ Wt[pre + "o"].T


def xielu(z, p, q):
    sp = math.log1p(math.exp(float(p)))
    sq = math.log1p(math.exp(float(q)))
    pos = sp * z * z + z / 2
    neg = (0.5 + sq) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def feed_forward(Wt, pre, h):
    z = h @ Wt[pre + "up"].T + Wt[pre + "up.b"]
    return xielu(z, Wt[pre + "act"][0], Wt[pre + "act"][1]) @ Wt[pre + "down"].T + Wt[pre + "down.b"]


def forward(config, Wt, tokens, residuals=None):
    """Logits [T, vocab] of one sequence; `residuals` (a list) receives x after every layer."""
    eps, alpha = config["norm"]["eps"], config["postln_alpha"]
    x = Wt["embed"][torch.tensor(tokens)]
    held = {}
    for n, layer in enumerate(config["layers"]):
        pre, m = f"l{n}.", layer["mixer"]
        h = shifted_conv(x, Wt[pre + "canon1"])
        if layer["type"] == "latent_attention":
            if "kv_from" in m:
                lat, key = held[m["kv_from"]]
            else:
                lat, key = held[n] = latent_kv(Wt, pre + "mix.", m, h, eps)
            y = latent_attention(Wt, pre + "mix.", m, h, lat, key, eps)
        else:
            y = delta_rule(Wt, pre + "mix.", m, h, eps)
        x = unit_rms(alpha * x + y, eps) * (1 + Wt[pre + "norm1"])
        if layer["mlp"] is not None:
            h = shifted_conv(x, Wt[pre + "canon2"])
            x = unit_rms(alpha * x + feed_forward(Wt, pre + "mlp.", h), eps) * (1 + Wt[pre + "norm2"])
        if residuals is not None:
            residuals.append(x.clone())
    return (unit_rms(x, eps) * (1 + Wt["final.norm"])) @ Wt["head"].T


def random_weights(config, seed, decay_rank=5):
    """bf16-representable random tensors under the checkpoint names, as fp64."""
    g = torch.Generator().manual_seed(seed)
    W, V, taps = config["width"], config["vocab"], config["canon"]["taps"]
    out = {}

    def mat(name, o, i, gain=1.0):
        out[name] = torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(name, n, std, mean=0.0):
        out[name] = torch.randn(n, generator=g) * std + mean
    out["embed"] = torch.randn(V, W, generator=g)
    mat("head", V, W)
    vec("final.norm", W, 0.2)
    for n, layer in enumerate(config["layers"]):
        pre, m = f"l{n}.", layer["mixer"]
        vec(pre + "norm1", W, 0.2)
        out[pre + "canon1"] = torch.randn(W, taps, generator=g) * 0.4
        if layer["type"] == "latent_attention":
            H, dn, dr, dv, R, Rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            mat(pre + "mix.dq", Rq, W)
            vec(pre + "mix.dq.norm", Rq, 0.2, 1.0)
            mat(pre + "mix.uq", H * (dn + dr), Rq, 2.0)
            if "kv_from" not in m:
                mat(pre + "mix.dkv", R + dr, W)
                vec(pre + "mix.dkv.norm", R, 0.2, 1.0)
            mat(pre + "mix.uk", H * dn, R, 2.0)
            mat(pre + "mix.uv", H * dv, R)
            mat(pre + "mix.g", H, W)
            mat(pre + "mix.o", W, H * dv)
        else:
            HD = m["heads"] * m["dim"]
            for nm in ("r", "k", "v", "g", "a"):
                mat(pre + "mix." + nm, HD, W)
            mat(pre + "mix.w1", decay_rank, W)
            mat(pre + "mix.w2", HD, decay_rank, 2.0)
            vec(pre + "mix.w0", HD, 1.0)
            vec(pre + "mix.a.b", HD, 0.5)
            vec(pre + "mix.norm", HD, 0.2, 1.0)
            mat(pre + "mix.o", W, HD)
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            vec(pre + "norm2", W, 0.2)
            out[pre + "canon2"] = torch.randn(W, taps, generator=g) * 0.4
            mat(pre + "mlp.up", ff, W)
            vec(pre + "mlp.up.b", ff, 0.2)
            mat(pre + "mlp.down", W, ff)
            vec(pre + "mlp.down.b", W, 0.2)
            vec(pre + "mlp.act", 2, 0.7)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in out.items()}


def write_checkpoint(path, config, Wt):
    import json
    import os

    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in Wt.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
