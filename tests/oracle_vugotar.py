"""A slow float64 whole-sequence oracle of the Vugotar decoder, one function per mechanism. It takes the configuration
as the plain dictionary of config.json and the tensors as a name -> tensor mapping, and shares no code with the
package: the tests compare the engine (cache, state slots, kernels, scheduler) with it.

Notation: T tokens of ONE sequence, positions 0 .. T-1; weights are [out, in] and applied as x @ W.T.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def d(t):
    return t.to(F64)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + d(w))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def rotary_pairs(x, pos, dims, base):
    """x [T, heads, dim]: neighbours (2i, 2i+1) of the first `dims` numbers of a head turn by pos * base^(-2i/dims)."""
    out = x.clone()
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = d(pos)[:, None] * f[None, :]  # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def chunk_sink_attention(q, k, v, scale, chunk):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv]. Token i sees j <= i of its own chunk (positions counted from 0 in
    blocks of `chunk`); the softmax denominator holds one extra term exp(0) that carries no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = (i // chunk) * chunk if chunk else 0
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = max(float(s.max()), 0.0)
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (math.exp(-m) + e.sum())
    return out


def causal_taps(x, w, bias=None):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the sequence starts."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        y += d(w)[:, j] * pad[j:j + T]
    if bias is not None:
        y = y + d(bias)
    return y


def delta_rule(q, k, v, beta, g):
    """Gated delta rule of one head. q, k [T, dk], v [T, dv], beta, g [T]. Returns o [T, dv]."""
    T, dk = q.shape
    S = torch.zeros(dk, v.shape[1], dtype=F64)
    o = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o


def left_mixer(m, W, p, h, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ d(W[p + "q"]).T).reshape(T, H, dk)
    k = (h @ d(W[p + "k"]).T).reshape(T, G, dk)
    v = (h @ d(W[p + "v"]).T).reshape(T, G, dv)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotary_pairs(q, pos, rot["dims"], rot["base"])
        k = rotary_pairs(k, pos, rot["dims"], rot["base"])
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    o = chunk_sink_attention(q, k, v, m["scale"], (m.get("mask") or {}).get("size", 0))
    return o.reshape(T, H * dv) @ d(W[p + "o"]).T


def right_mixer(m, W, p, h, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_taps(h @ d(W[p + "q"]).T, W[p + "q.conv"])).reshape(T, G, dk)
    k = silu(causal_taps(h @ d(W[p + "k"]).T, W[p + "k.conv"])).reshape(T, G, dk)
    v = silu(causal_taps(h @ d(W[p + "v"]).T, W[p + "v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ d(W[p + "b"]).T)  # [T, H]
    g = torch.exp(-torch.exp(d(W[p + "A_log"])) * softplus(h @ d(W[p + "a"]).T + d(W[p + "dt_bias"])))
    gate = silu(h @ d(W[p + "g"]).T).reshape(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        kv = hd // (H // G)
        o[:, hd] = delta_rule(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], g[:, hd])
    o = unit_rms(o, eps) * d(W[p + "norm"]) * gate
    return o.reshape(T, H * dv) @ d(W[p + "o"]).T


def parallel_mixer(m, W, p, h, eps):
    return m["left_scale"] * left_mixer(m["left"], W, p + "left.", h, eps) + \
        m["right_scale"] * right_mixer(m["right"], W, p + "right.", h, eps)


def mamba2_mixer(m, W, p, h, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    y = h @ d(W[p + "in"]).T
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_taps(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + d(W[p + "dt_bias"]))  # [T, H]
    A = torch.exp(d(W[p + "A_log"]))
    D = d(W[p + "D"])
    out = torch.zeros(T, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(-A[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            out[t, hd] = S.T @ C[t, g] + D[hd] * x[t, hd]
    out = out.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    out = unit_rms(out.reshape(T, ng, inner // ng), eps).reshape(T, inner) * d(W[p + "norm"])
    return out @ d(W[p + "o"]).T


def glu_ffn(W, p, h, biased):
    a = h @ d(W[p + "gate"]).T
    b = h @ d(W[p + "up"]).T
    if biased:
        a, b = a + d(W[p + "gate.b"]), b + d(W[p + "up.b"])
    y = (silu(a) * b) @ d(W[p + "down"]).T
    return y + d(W[p + "down.b"]) if biased else y


def moe_ffn(mlp, W, p, h):
    r = mlp["router"]
    s = torch.softmax(h @ d(W[p + "router"]).T, -1)
    top = torch.topk(s, r["top"], dim=-1)
    wts = top.values / (top.values.sum(-1, keepdim=True) + 1e-20) * r["scale"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(r["top"]):
            e = int(top.indices[t, j])
            out[t] += wts[t, j] * glu_ffn(W, f"{p}e{e}.", h[t:t + 1], False)[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ d(W[p + "shared.sg"]).T) * glu_ffn(W, p + "shared.", h, False)
    return out


def feed_forward(mlp, W, p, h):
    if mlp is None:
        return torch.zeros_like(h)
    if mlp["kind"] == "dense":
        return glu_ffn(W, p, h, True)
    if mlp["kind"] == "moe":
        return moe_ffn(mlp, W, p, h)
    raise ValueError(mlp["kind"])


def layer_order(cfg):
    """Indices of the layers in the order they run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp.get("times", 1) <= 1:
        return [(i, False) for i in range(n)]
    a, b, k = lp["start"], lp["stop"], lp["times"]
    order = [(i, False) for i in range(a)]
    for r in range(k):
        order += [(i, r > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens):
    """Logits [T, vocab] and the residual after every layer run [runs, T, width] of one whole sequence."""
    eps = cfg["norm"]["eps"]
    x0 = d(W["embed"])[torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    trace = []
    for i, add_embed in layer_order(cfg):
        L = cfg["layers"][i]
        if add_embed:
            x = x + x0
        h = offset_norm(x, W[f"l{i}.norm1"], eps)
        if L["type"] == "parallel":
            mix = parallel_mixer(L["mixer"], W, f"l{i}.mix.", h, eps)
        elif L["type"] == "mamba2":
            mix = mamba2_mixer(L["mixer"], W, f"l{i}.mix.", h, eps)
        else:
            raise ValueError(L["type"])
        x = x + (mix + feed_forward(L.get("mlp"), W, f"l{i}.mlp.", h))
        trace.append(x.clone())
    logits = offset_norm(x, W["final.norm"], eps) @ d(W["head"]).T
    return logits, torch.stack(trace)
