"""Plain whole-sequence oracle of the Vosotar decoder, one function per mechanism, in float64 on the CPU.

It takes the checkpoint's tensors by name (a dict of torch tensors) and the configuration dict, runs one
sequence from position 0 with no cache and no batching, and shares no code with the package: the tests
compare the engine (paged latent cache, carried convolution tails, ragged batches, HIP kernels) with it.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return unit_rms(x, eps) * g.to(F64).reshape(())


def vector_norm(x, w, eps):
    """RMS norm with one gain per coordinate."""
    return unit_rms(x, eps) * w.to(F64)


def tap_conv(h, w):
    """y_t = sum_j w[:, j] * h_(t - taps + 1 + j) on each channel, zeros before the first row. h [n, C], w [C, taps]."""
    n, taps = h.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, h.shape[1], dtype=F64), h], 0)
    y = torch.zeros_like(h)
    for j in range(taps):
        y += w[:, j].to(F64) * pad[j:j + n]
    return y


def latent_attention(h, t, p, m, eps):
    """Causal softmax attention whose keys and values are both expanded from one normed latent per token.
    h [n, C]; t: tensors; p: tensor-name prefix of the mixer; m: its sizes."""
    H, d, dv, scale = m["heads"], m["dim"], m["vdim"], float(m["scale"])
    n = h.shape[0]
    W = lambda k: t[p + k].to(F64)  # noqa: E731
    cq = vector_norm(h @ W("dq").T, t[p + "dq.norm"], eps)
    q = (cq @ W("uq").T).reshape(n, H, d)
    c = vector_norm(h @ W("dkv").T, t[p + "dkv.norm"], eps)
    k = (c @ W("uk").T).reshape(n, H, d)
    v = (c @ W("uv").T).reshape(n, H, dv)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    vis = torch.arange(n)[None, :] <= torch.arange(n)[:, None]
    s = s.masked_fill(~vis[None], -math.inf)
    a = torch.softmax(s, -1)
    o = torch.einsum("hij,jhe->ihe", a, v)
    o = o * torch.sigmoid(h @ W("g").T)[:, :, None]
    return o.reshape(n, H * dv) @ W("o").T


def relu2_ffn(h, t, p):
    u = torch.relu(h @ t[p + "up"].to(F64).T)
    return (u * u) @ t[p + "down"].to(F64).T


def sublayer_gate(h, t, name):
    return torch.sigmoid(h @ t[name].to(F64).T + t[name + ".b"].to(F64))


def layer(x, t, src: str, entry: dict, eps: float):
    """One layer on the residual x [n, C]; `src` is the prefix of the layer whose tensors it uses."""
    h = scalar_norm(x, t[src + "norm1"], eps)
    gate = sublayer_gate(h, t, src + "rg1")
    hm = h + tap_conv(h, t[src + "canon1"])
    if entry["type"] != "latent_attention":
        raise ValueError(entry["type"])
    y = latent_attention(hm, t, src + "mix.", entry["mixer"], eps) * gate
    x = x + scalar_norm(y, t[src + "norm1b"], eps)
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "dense":
            raise ValueError(entry["mlp"]["kind"])
        h = scalar_norm(x, t[src + "norm2"], eps)
        y = relu2_ffn(h, t, src + "mlp.") * sublayer_gate(h, t, src + "rg2")
        x = x + scalar_norm(y, t[src + "norm2b"], eps)
    return x


def forward(cfg: dict, t: dict, tokens, return_layers: bool = False):
    """Logits [n, vocab] of one sequence (and the residual after every layer run when asked)."""
    eps = float(cfg["norm"]["eps"])
    x = scalar_norm(t["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)], t["embed.norm"], eps)
    outs = []
    for i, e in enumerate(cfg["layers"]):
        x = layer(x, t, "l%d." % e.get("weights_of", i), e, eps)
        outs.append(x)
    logits = scalar_norm(x, t["final.norm"], eps) @ t["head"].to(F64).T
    return (logits, torch.stack(outs)) if return_layers else logits
