"""Plain, slow restatement of the Vumalix decoder in torch on the CPU, one function per mechanism.  Test infrastructure only:
nothing under ``jacobiforcing_amd/`` imports it and it shares no code with the package.  Every function works on ONE whole
sequence (tokens 0 .. T-1) in the dtype of its inputs (float32 or float64) and has no cache: position t simply sees what its
mask lets it see.  Latent attention is written the long way round — keys and values are built from every token's latent — where
the package multiplies the query by the key up-projection instead.

Notation: ``h`` [T, width] what a mixer reads, ``P`` a dict of a layer's tensors keyed by the name behind ``l<i>.`` (``mix.q``,
``mlp.up`` …), ``m`` the layer's ``mixer`` entry of config.json."""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def time_conv_mix(x, w):
    """x [T, width], w [width, taps]: y_t = x_t + sum_j w[:, j] * x_(t - taps + 1 + j), nothing before t = 0."""
    T, taps = x.shape[0], w.shape[1]
    y = x.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * x[s]
    return y


def rotate_pairs(vec, position: int, dims: int, base: float):
    """vec [.., d]: of the first ``dims`` entries, i and i + dims/2 are a pair turned by position * base^(-2i/dims); angles in float32."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float32)
    a = torch.tensor(float(position), dtype=torch.float32) * f
    c, s = torch.cos(a).to(vec.dtype), torch.sin(a).to(vec.dtype)
    u, v = vec[..., :half], vec[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, vec[..., dims:]], -1)


def query_temperature(position: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((position + 1) // every + 1)


def differential_lambda(P, diff: float):
    return float(torch.exp((P["mix.lq1"] * P["mix.lk1"]).sum()) - torch.exp((P["mix.lq2"] * P["mix.lk2"]).sum()) + diff)


def differential_attention(h, P, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    qt = m.get("q_temp") or {"coef": 0.0, "every": 1}
    q = unit_rms((h @ P["mix.q"].T).view(T, H, 2, D), eps) * P["mix.q.norm"]
    k = unit_rms((h @ P["mix.k"].T).view(T, G, 2, D), eps) * P["mix.k.norm"]
    v = (h @ P["mix.v"].T).view(T, G, Dv)
    lam = differential_lambda(P, m["diff"])
    size = (m.get("mask") or {}).get("size", 0) or T + 1           # the design's layers have no window; one that has is honoured
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(T):
        temp = query_temperature(i, qt["coef"], qt["every"])
        lo = max(0, i - size + 1)
        for hh in range(H):
            c = hh // (H // G)
            maps = []
            for mp in range(2):
                s = (k[lo:i + 1, c, mp] @ (q[i, hh, mp] * temp)) * m["scale"]
                maps.append(torch.softmax(s, 0) @ v[lo:i + 1, c])
            o = maps[0] - lam * maps[1]
            out[i, hh] = unit_rms(o, eps) * (1.0 - m["diff"])
    return out.reshape(T, H * Dv) @ P["mix.o"].T


def latent_attention(h, P, m, eps):
    T = h.shape[0]
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    dims, base = m["rot"]["dims"], m["rot"]["base"]
    size = (m.get("mask") or {}).get("size", 0) or T + 1
    q = ((unit_rms(h @ P["mix.dq"].T, eps) * P["mix.dq.norm"]) @ P["mix.uq"].T).view(T, H, D + rd)
    down = h @ P["mix.dkv"].T
    latent = unit_rms(down[:, :R], eps) * P["mix.dkv.norm"]
    k_plain = (latent @ P["mix.uk"].T).view(T, H, D)
    value = (latent @ P["mix.uv"].T).view(T, H, Dv)
    k_turn = torch.stack([rotate_pairs(down[t, R:], t, dims, base) for t in range(T)])          # [T, rd], one for all heads
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            q_turn = rotate_pairs(q[i, hh, D:], i, dims, base)
            s = (k_plain[lo:i + 1, hh] @ q[i, hh, :D] + k_turn[lo:i + 1] @ q_turn) * m["scale"]
            out[i, hh] = torch.softmax(s, 0) @ value[lo:i + 1, hh]
    gate = torch.sigmoid(h @ P["mix.g"].T)
    return (out.reshape(T, H * Dv) * gate) @ P["mix.o"].T


def polynomial_activation(z, coef, eps):
    return coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z * z, eps) + coef[2] * unit_rms(z * z * z, eps) + coef[3]


def feed_forward(h, P, eps):
    return polynomial_activation(h @ P["mlp.up"].T, P["mlp.act"], eps) @ P["mlp.down"].T


def layer_tensors(tensors, i: int):
    p = f"l{i}."
    return {k[len(p):]: v for k, v in tensors.items() if k.startswith(p)}


def forward(cfg, tensors, tokens, dtype=torch.float64):
    """Logits [T, vocab] and the residual stream after every layer [layers, T, width] for one whole sequence."""
    eps = cfg["norm"]["eps"]
    x = tensors["embed"].to(dtype)[torch.tensor(list(tokens))]
    trace = []
    for i, L in enumerate(cfg["layers"]):
        P = {k: v.to(dtype) for k, v in layer_tensors(tensors, L.get("weights_of", i)).items()}
        h = time_conv_mix(x, P["canon1"])
        y = differential_attention(h, P, L["mixer"], eps) if L["type"] == "attention" else latent_attention(h, P, L["mixer"], eps)
        x = x + unit_rms(y, eps) * P["norm1"]
        if L.get("mlp") is not None:
            x = x + unit_rms(feed_forward(x, P, eps), eps) * P["norm2"]
        trace.append(x.clone())
    logits = (unit_rms(x, eps) * tensors["final.norm"].to(dtype)) @ tensors["head"].to(dtype).T
    return logits, torch.stack(trace)
