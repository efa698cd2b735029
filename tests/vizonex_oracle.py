"""Slow, dense, fp64 oracle of the Vizonex design: one function per mechanism, whole sequences,
no cache, no batching. It shares nothing with xgserve's model or ops; the tests compare the
framework against it. Weights are a dict of checkpoint tensor names -> fp64 tensors.

Notation: x_t is the residual row of token t (t = 0 is the sequence's first token); a layer is
x_t <- x_t + a1 * mixer(n_t + conv(n)_t) + a2 * ff(n_t)  with  n_t = rmsnorm(x_t) * g.
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------ small pieces
def unit_rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def shifted_conv(h, w, bias=None):
    """sum_j w[:, j] h_(t - taps + 1 + j) (+ bias); rows before t = 0 are zero. h [T, C], w [C, taps]."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
        if bias is not None:
            out[t] += bias
    return out


# ------------------------------------------------------------------------------ attention in chunks, with a sink
def chunk_softmax(q, k, v, size, scale, temp, sink):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] of one sequence -> [T, H, dv]. Query i reads keys j <= i of its
    own chunk floor(i / size); the denominator carries exp(sink_h) besides the keys' terms."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            lo = (i // size) * size
            s = (k[lo:i + 1, g] @ q[i, hd]) * scale * temp[hd]
            top = torch.maximum(s.max(), sink[hd])
            e = torch.exp(s - top)
            out[i, hd] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (e.sum() + torch.exp(sink[hd] - top))
    return out


def chunk_attention(Wt, pre, m, h, eps):
    """Whole-vector query / key norms, no positional rotation, per-head temperature, keys of the
    query's own chunk only (chunks of m.mask.size counted from t = 0), and one extra term
    exp(sink_h) in the softmax denominator that carries no value."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms(h @ Wt[pre + "q"].T, eps) * Wt[pre + "q.norm"]
    k = unit_rms(h @ Wt[pre + "k"].T, eps) * Wt[pre + "k.norm"]
    v = h @ Wt[pre + "v"].T
    out = chunk_softmax(q.reshape(T, H, dk), k.reshape(T, G, dk), v.reshape(T, G, dv), int(m["mask"]["size"]),
                        float(m["scale"]), Wt[pre + "temp"], Wt[pre + "sink"])
    return out.reshape(T, H * dv) @ Wt[pre + "o"].T


# ------------------------------------------------------------------------------ state-space recurrence
def ssm_mixer(Wt, pre, m, h, eps, states=None):
    """Selective state-space layer with a scalar decay per head:
    S_t = exp(-exp(A_h) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + D_h x_t."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, ng = H * P, m["norm_groups"]
    proj = h @ Wt[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == H
    xbc = silu(shifted_conv(xbc, Wt[pre + "conv"], Wt[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + Wt[pre + "dt_bias"])
    y = torch.zeros(T, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        rate = torch.exp(Wt[pre + "A_log"][hd])
        for t in range(T):
            S = torch.exp(-rate * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + Wt[pre + "D"][hd] * x[t, hd]
        if states is not None:
            states.append(S)
    y = y.reshape(T, inner) * silu(z)
    y = unit_rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * Wt[pre + "norm"]
    return y @ Wt[pre + "o"].T


# ------------------------------------------------------------------------------ feed-forward
def dense_ff(Wt, pre, h):
    return (gelu_tanh(h @ Wt[pre + "gate"].T) * (h @ Wt[pre + "up"].T)) @ Wt[pre + "down"].T


def clamped_expert(Wt, pre, h, limit):
    g = torch.clamp(h @ Wt[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ Wt[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ Wt[pre + "down"].T


def route_scores(z, correction, r):
    """Router logits z [T, E] -> per row the chosen experts and their weights: lists of (expert, weight)."""
    E, top = r["experts"], r["top"]
    count, keep = r["groups"]["count"], r["groups"]["keep"]
    s = torch.sigmoid(z)
    pick = s + correction
    per = E // count
    chosen = []
    for t in range(z.shape[0]):
        gs = []
        for g in range(count):
            part = sorted(pick[t, g * per:(g + 1) * per].tolist(), reverse=True)
            gs.append(sum(part[:2]))
        kept = sorted(range(count), key=lambda g: -gs[g])[:keep]
        cand = [e for e in range(E) if e // per in kept]
        cand.sort(key=lambda e: -float(pick[t, e]))
        chosen.append([(e, float(s[t, e]) * r["scale"]) for e in cand[:top]])
    return chosen


def route(Wt, pre, r, h):
    return route_scores(h @ Wt[pre + "router"].T, Wt[pre + "correction"], r)


def moe_ff(Wt, pre, mlp, h):
    out = torch.zeros(h.shape[0], Wt[pre + "e0.down"].shape[0], dtype=F64)
    for t, sel in enumerate(route(Wt, pre, mlp["router"], h)):
        for e, w in sel:
            out[t] += w * clamped_expert(Wt, f"{pre}e{e}.", h[t:t + 1], mlp["expert"]["limit"])[0]
    if mlp.get("shared") is not None:
        out += clamped_expert(Wt, pre + "shared.", h, mlp["shared"]["limit"])
    return out


# ------------------------------------------------------------------------------ whole model
def layer_forward(config, Wt, n, x):
    layer = config["layers"][n]
    pre, eps = f"l{n}.", config["norm"]["eps"]
    nrm = unit_rms(x, eps) * Wt[pre + "norm1"]
    hm = nrm + shifted_conv(nrm, Wt[pre + "canon1"])
    if layer["type"] == "attention":
        y = chunk_attention(Wt, pre + "mix.", layer["mixer"], hm, eps)
    elif layer["type"] == "mamba2":
        y = ssm_mixer(Wt, pre + "mix.", layer["mixer"], hm, eps)
    else:
        raise ValueError(layer["type"])
    x = x + y * Wt[pre + "ls1"]
    mlp = layer.get("mlp")
    if mlp is not None:
        f = dense_ff(Wt, pre + "mlp.", nrm) if mlp["kind"] == "dense" else moe_ff(Wt, pre + "mlp.", mlp, nrm)
        x = x + f * Wt[pre + "ls2"]
    return x


def forward(config, Wt, tokens, residuals=None):
    """Logits [T, vocab] of one sequence; `residuals` (a list) receives x after every layer."""
    T = len(tokens)
    x = Wt["embed"][torch.tensor(tokens)] + Wt["pos"][:T]
    for n in range(len(config["layers"])):
        x = layer_forward(config, Wt, n, x)
        if residuals is not None:
            residuals.append(x.clone())
    return (unit_rms(x, config["norm"]["eps"]) * Wt["final.norm"]) @ Wt["head"].T


# ------------------------------------------------------------------------------ test models
def random_weights(config, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, V, taps = config["width"], config["vocab"], config["canon"]["taps"]
    out = {}

    def mat(name, o, i, gain=1.0):
        out[name] = torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(name, n, std, mean=0.0):
        out[name] = torch.randn(n, generator=g) * std + mean

    def expert(pre, ff):
        mat(pre + "gate", ff, W, 2.0)
        mat(pre + "up", ff, W, 2.0)
        mat(pre + "down", W, ff)
    out["embed"] = torch.randn(V, W, generator=g)
    out["pos"] = torch.randn(config["max_positions"], W, generator=g) * 0.5
    mat("head", V, W)
    vec("final.norm", W, 0.2, 1.0)
    for n, layer in enumerate(config["layers"]):
        pre, m = f"l{n}.", layer["mixer"]
        vec(pre + "norm1", W, 0.2, 1.0)
        vec(pre + "ls1", W, 0.2, 0.7)
        out[pre + "canon1"] = torch.randn(W, taps, generator=g) * 0.4
        if layer["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(pre + "mix.q", H * dk, W)
            mat(pre + "mix.k", G * dk, W)
            mat(pre + "mix.v", G * dv, W)
            vec(pre + "mix.q.norm", H * dk, 0.3, 1.5)
            vec(pre + "mix.k.norm", G * dk, 0.3, 1.5)
            vec(pre + "mix.temp", H, 0.3, 1.2)
            vec(pre + "mix.sink", H, 1.0, 0.5)
            mat(pre + "mix.o", W, H * dv)
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = H * P + 2 * G * N
            mat(pre + "mix.in", 2 * H * P + 2 * G * N + H, W)
            out[pre + "mix.conv"] = torch.randn(ch, m["conv"], generator=g) * 0.5
            vec(pre + "mix.conv.b", ch, 0.2)
            vec(pre + "mix.dt_bias", H, 0.5, -1.0)
            vec(pre + "mix.A_log", H, 0.5, -0.5)
            vec(pre + "mix.D", H, 0.5, 1.0)
            vec(pre + "mix.norm", H * P, 0.2, 1.0)
            mat(pre + "mix.o", W, H * P)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        vec(pre + "ls2", W, 0.2, 0.7)
        if mlp["kind"] == "dense":
            expert(pre + "mlp.", mlp["ff"])
        else:
            E = mlp["router"]["experts"]
            for e in range(E):
                expert(f"{pre}mlp.e{e}.", mlp["expert"]["ff"])
            mat(pre + "mlp.router", E, W, 2.0)
            vec(pre + "mlp.correction", E, 0.3)
            if mlp.get("shared") is not None:
                expert(pre + "mlp.shared.", mlp["shared"]["ff"])
    return {k: v.to(torch.bfloat16).to(F64) for k, v in out.items()}


def write_checkpoint(path, config, Wt):
    import json
    import os

    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in Wt.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
