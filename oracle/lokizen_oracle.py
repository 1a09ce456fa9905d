"""Plain, slow restatement of the Lokizen decoder in torch on the CPU, one function per mechanism.  Test infrastructure only:
nothing under ``jacobiforcing_amd/`` imports it and it shares no code with the package.  Every function works on ONE whole
sequence (tokens 0 .. T-1) in the dtype of its inputs (float32 or float64) and has no cache: position t simply sees what its
mask lets it see.

Notation: ``h`` [T, width] the mixer / feed-forward input, ``P`` a dict of a layer's tensors keyed by the name behind
``l<i>.`` (``mix.q``, ``mlp.e3.up`` …), ``m`` the layer's ``mixer`` / ``mlp`` entry of config.json."""
from __future__ import annotations

import math

import torch


def rms_norm(x, w=None, eps=1e-5):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance-bias table for distance n >= 0: one row per distance below rows/2, logarithmic steps from there up
    to ``far``, the last row beyond."""
    half = rows // 2
    if n < half:
        return n
    import numpy as np
    f = np.float32
    step = np.log(f(n) / f(half)) / np.log(f(far) / f(half)) * f(rows - half)
    return min(rows - 1, half + int(math.floor(float(step))))


def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def attention_mixer(h, P, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ P["mix.q"].T, P["mix.q.norm"], eps).view(T, H, D)
    k = rms_norm(h @ P["mix.k"].T, P["mix.k.norm"], eps).view(T, G, D)
    v = (h @ P["mix.v"].T).view(T, G, Dv)
    rel, talk = P["mix.rel"], P["mix.talk"]
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    rows = rel.shape[0]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(T):
        js = [j for j in range(i + 1) if visible(i, j, size, keep)]
        w = torch.zeros(H, len(js), dtype=h.dtype)
        for g in range(H):
            c = g // (H // G)
            s = torch.stack([(q[i, g] * k[j, c]).sum() * m["scale"] + rel[distance_bucket(i - j, rows, m["bias_max"]), g] for j in js])
            w[g] = torch.softmax(s, 0)
        w = talk @ w                                            # head h's weights: sum_g talk[h, g] w_g
        for hh in range(H):
            c = hh // (H // G)
            out[i, hh] = (w[hh].view(-1, 1) * v[js, c]).sum(0)
    gate = torch.sigmoid(h @ P["mix.g"].T)
    return (out.reshape(T, H * Dv) * gate) @ P["mix.o"].T


def rotate_half_pairs(x, dims, base):
    """x [T, heads, D]: dimension i < dims/2 pairs with i + dims/2; angle = position * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float32)
    a = torch.arange(T, dtype=torch.float32).view(T, 1) * f.view(1, half)
    cos, sin = torch.cos(a).to(x.dtype).view(T, 1, half), torch.sin(a).to(x.dtype).view(T, 1, half)
    u, w = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - w * sin, w * cos + u * sin, x[..., dims:]], -1)


def retention_mixer(h, P, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = rotate_half_pairs((h @ P["mix.q"].T).view(T, H, D), m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half_pairs((h @ P["mix.k"].T).view(T, H, D), m["rot"]["dims"], m["rot"]["base"]) * D ** -0.5
    v = (h @ P["mix.v"].T).view(T, H, Dv)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    decay = torch.tensor(m["decay"], dtype=h.dtype).view(H, 1, 1)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        S = decay * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = (S * q[t].unsqueeze(-1)).sum(1)
    o = rms_norm(o, None, eps).reshape(T, H * Dv)
    g = h @ P["mix.g"].T
    return (o * (g * torch.sigmoid(g))) @ P["mix.o"].T


def moe_feed_forward(h, P, m):
    r = m["router"]
    s = torch.sigmoid(h @ P["mlp.router"].T)
    choice = s + P["mlp.correction"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(choice[t], r["top"]).indices.tolist()
        for e in chosen:
            a = torch.relu(P[f"mlp.e{e}.up"] @ h[t]) ** 2
            out[t] += s[t, e] * r["scale"] * (P[f"mlp.e{e}.down"] @ a)
    return out


def layer_runs(cfg):
    """(layer index, first layer of a repeated pass?) in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    runs = [(i, False) for i in range(lp["start"])]
    for p in range(lp["times"]):
        runs += [(i, p > 0 and i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return runs + [(i, False) for i in range(lp["stop"], n)]


def layer_tensors(W, i):
    pre = f"l{i}."
    return {k[len(pre):]: v for k, v in W.items() if k.startswith(pre)}


def forward(cfg, W, tokens, dtype=torch.float32):
    """logits [T, vocab] and the residual stream after every layer run [runs, T, width]."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x0 = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    x = x0.clone()
    trace = []
    for i, readd in layer_runs(cfg):
        L, P = cfg["layers"][i], layer_tensors(W, i)
        if readd:
            x = x + x0
        hn = rms_norm(x, P["norm1"], eps)
        x = x + (attention_mixer(hn, P, L["mixer"], eps) if L["type"] == "attention" else retention_mixer(hn, P, L["mixer"], eps))
        if L.get("mlp"):
            x = x + moe_feed_forward(rms_norm(x, P["norm2"], eps), P, L["mlp"])
        trace.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T, torch.stack(trace)
