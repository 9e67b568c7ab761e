"""Ops of decoders that cache one low-rank latent per token instead of keys and values, plus the small sequence-state
ops such decoders combine with it: a scalar-gain RMS norm, a causal per-channel tap convolution whose last inputs
are carried per sequence, a sigmoid-gated and normed residual add, and the squared-ReLU activation.

Latent attention (weight-absorbed form). A layer projects each token to a normed latent c_j of `rank` numbers; keys
and values are linear in it (k_j = U_k c_j, v_j = U_v c_j per head). With qa = U_k^T q per head the score is
qa . c_j, and the head's output is U_v (sum_j p_j c_j): the kernels therefore run an attention whose keys and values
are BOTH the cached latents, shared by all heads, and the caller applies U_k^T before and U_v after as batched
GEMMs. Only the latent is cached: a paged pool [blocks, block_size, rank] per layer (engine/kv_cache.py LatentCache).

Every function runs the HIP kernels of csrc/kernels/latent/ on GPU tensors and a plain fp32 PyTorch form on CPU
tensors (the plumbing path of GPU-less environments). Norms, softmax, scores and the residual are fp32 in both;
16-bit tensors appear only as GEMM operands and as the cached latent.
"""
from __future__ import annotations

import torch

from .. import _native as N


class Ragged:
    """Sequence layout of one engine step: `n_dec` single-token rows, then `n_pf` chunks whose row offsets
    (relative to the first chunk row) are `pf_cu`. `state` gives each sequence's state slot (decode rows first),
    `positions` each row's position in its sequence. Host copies serve the CPU path only."""

    def __init__(self, fb):
        self.T = fb.T
        self.n_dec = fb.n_decode
        self.pf_cu = fb.pf_cu_q
        self.n_pf = 0 if fb.pf_cu_q is None else int(fb.pf_cu_q.numel()) - 1
        self.positions = fb.positions
        self.slots = fb.slots
        self.state = fb.seq_state
        self.dec_bt, self.dec_lens = fb.dec_block_tables, fb.dec_seq_lens
        self.pf_bt, self.pf_ctx = fb.pf_block_tables, fb.pf_ctx_lens
        self.dec_max_len = fb.dec_max_len
        # rows and context length of each chunk on the host (empty when the step replays a captured graph)
        self.pf_q_host = list(getattr(fb, "pf_q_lens_host", None) or [])
        self.pf_ctx_host = list(getattr(fb, "pf_ctx_lens_host", None) or [])

    def host_segments(self):
        """[(first row, rows, index into `state`)] on the host."""
        out = [(i, 1, i) for i in range(self.n_dec)]
        if self.n_pf:
            cu = self.pf_cu.tolist()
            out += [(self.n_dec + cu[k], cu[k + 1] - cu[k], self.n_dec + k) for k in range(self.n_pf)
                    if cu[k + 1] > cu[k]]
        return out


def _is16(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise TypeError(f"latent ops take float32 or bfloat16 tensors, not {t.dtype}")


# ------------------------------------------------------------------------------------------------ norms
def embed_scalar_norm(table: torch.Tensor, tokens: torch.Tensor, g: torch.Tensor, eps: float, out: torch.Tensor):
    """out[t] = unit_rms(table[tokens[t]]) * g, g one number; out fp32 [T, C]."""
    T, C = out.shape
    if T == 0:
        return out
    if not out.is_cuda:
        x = table[tokens.long()].float()
        out.copy_(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * g.float())
        return out
    N.kcall("mxl_embed_norm", table.data_ptr(), _is16(table), table.shape[0], tokens.data_ptr(), g.data_ptr(),
            float(eps), out.data_ptr(), out.stride(0), T, C, N.stream_ptr())
    return out


def scalar_rmsnorm(x: torch.Tensor, g: torch.Tensor, eps: float, out32: torch.Tensor | None = None,
                   out16: torch.Tensor | None = None, rows: torch.Tensor | None = None):
    """y = unit_rms(x) * g for fp32 rows (g a one-element fp32 tensor), written as fp32 and / or bf16.
    `rows` (int32) picks the rows of x to norm: output row i comes from x[rows[i]]."""
    M = int(rows.numel()) if rows is not None else x.shape[0]
    C = x.shape[1]
    if M == 0:
        return
    if not x.is_cuda:
        xs = x[rows.long()] if rows is not None else x
        y = xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps) * g.float()
        if out32 is not None:
            out32.copy_(y)
        if out16 is not None:
            out16.copy_(y)
        return
    N.kcall("mxl_scalar_norm", x.data_ptr(), x.stride(0), N.ptr(rows), g.data_ptr(), float(eps), N.ptr(out32),
            out32.stride(0) if out32 is not None else 0, N.ptr(out16), out16.stride(0) if out16 is not None else 0,
            M, C, N.stream_ptr())


def gated_norm_add(x: torch.Tensor, y: torch.Tensor, gate_pre: torch.Tensor, g: torch.Tensor, eps: float,
                   gate_bias: torch.Tensor | None = None, next_g: torch.Tensor | None = None,
                   next32: torch.Tensor | None = None, next16: torch.Tensor | None = None):
    """x += unit_rms(y * sigmoid(gate_pre + gate_bias)) * g on fp32 rows [M, C]; gate_pre may be a column slice,
    gate_bias is fp32 [C]. With `next_g` the same pass also writes the following scalar-gain norm of the updated
    rows, next_g * unit_rms(x), as fp32 (`next32`) and / or bf16 (`next16`)."""
    M, C = y.shape
    if M == 0:
        return x
    if not x.is_cuda:
        gp = gate_pre.float() + gate_bias if gate_bias is not None else gate_pre.float()
        z = y.float() * torch.sigmoid(gp)
        x.add_(z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * g.float())
        if next_g is not None:
            scalar_rmsnorm(x, next_g, eps, out32=next32, out16=next16)
        return x
    N.kcall("mxl_gated_norm_add", x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), gate_pre.data_ptr(),
            gate_pre.stride(0), N.ptr(gate_bias), g.data_ptr(), float(eps), M, C, N.ptr(next_g), N.ptr(next32),
            next32.stride(0) if next32 is not None else 0, N.ptr(next16),
            next16.stride(0) if next16 is not None else 0, N.stream_ptr())
    return x


def relu2(u: torch.Tensor, out: torch.Tensor):
    """out = relu(u)^2; u fp32 [M, F] (may be a column slice), out fp32 or bf16 [M, F]."""
    M, F_ = out.shape
    if M == 0:
        return out
    if not u.is_cuda:
        r = torch.relu(u.float())
        out.copy_(r * r)
        return out
    N.kcall("mxl_relu2", u.data_ptr(), u.stride(0), out.data_ptr(), out.stride(0), _is16(out), M, F_, N.stream_ptr())
    return out


# ------------------------------------------------------------------------------------------------ tap convolution
def tap_conv(h: torch.Tensor, w: torch.Tensor, tails: torch.Tensor, rag: Ragged, out: torch.Tensor):
    """out = h + conv(h): conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j) per channel over each sequence's rows,
    with the sequence's previous taps - 1 inputs read from (and its newest ones written back to) `tails`
    [slots, taps - 1, C] fp32; a chunk that starts at position 0 reads zeros. h fp32 [T, C], w fp32 [C, taps];
    out fp32 or bf16. A state slot < 0 (padding rows) reads zeros and stores nothing."""
    T, C = h.shape
    taps = w.shape[1]
    if T == 0:
        return out
    if not h.is_cuda:
        st, pos = rag.state.tolist(), rag.positions.tolist()
        for r0, n, si in rag.host_segments():
            slot = st[si]
            fresh = pos[r0] == 0 or slot < 0 or taps == 1
            prev = torch.zeros(taps - 1, C) if fresh else tails[slot].clone()
            full = torch.cat([prev, h[r0:r0 + n].float()], 0)
            y = h[r0:r0 + n].float().clone()
            for j in range(taps):
                y += w[:, j] * full[j:j + n]
            out[r0:r0 + n] = y.to(out.dtype)
            if slot >= 0 and taps > 1:
                tails[slot] = full[full.shape[0] - (taps - 1):]
        return out
    if taps > 16:
        raise ValueError("tap_conv: at most 16 taps")
    N.kcall("mxl_tap_conv", h.data_ptr(), h.stride(0), w.data_ptr(), taps, tails.data_ptr(), rag.state.data_ptr(),
            rag.positions.data_ptr(), rag.n_dec, N.ptr(rag.pf_cu), rag.n_pf, out.data_ptr(), out.stride(0), _is16(out),
            T, C, N.stream_ptr())
    return out


# ------------------------------------------------------------------------------------------------ latents
def latent_norm_append(y: torch.Tensor, q_rank: int, rank: int, wq: torch.Tensor, wkv: torch.Tensor, eps: float,
                       cq: torch.Tensor, cache: torch.Tensor, slots: torch.Tensor):
    """Rows y [T, >= q_rank + rank] fp32 hold the query latent then the key/value latent. Writes
    cq = unit_rms(y[:, :q_rank]) * wq (fp32 or bf16 [T, q_rank]) and stores unit_rms(y[:, q_rank:q_rank + rank]) * wkv
    into the paged pool `cache` [blocks, block_size, rank] at flat slot slots[t] (slot < 0: not stored)."""
    T = y.shape[0]
    if T == 0:
        return
    if not y.is_cuda:
        a = y[:, :q_rank].float()
        cq.copy_(a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + eps) * wq)
        b = y[:, q_rank:q_rank + rank].float()
        c = b * torch.rsqrt(b.pow(2).mean(-1, keepdim=True) + eps) * wkv
        ok = slots >= 0
        cache.view(-1, rank)[slots[ok].long()] = c[ok].to(cache.dtype)
        return
    N.kcall("mxl_latent_norm_append", y.data_ptr(), y.stride(0), q_rank, rank, wq.data_ptr(), wkv.data_ptr(),
            float(eps), cq.data_ptr(), cq.stride(0), _is16(cq), cache.data_ptr(), _is16(cache), slots.data_ptr(), T,
            N.stream_ptr())


def _latent_attn_ref(qa, cache, table, ctx: int, pos0: int, scale: float, out):
    """qa [H, n, R], out [H, n, R]: rows at positions pos0.. of a sequence holding ctx cached latents."""
    bs, R = cache.shape[1], cache.shape[2]
    nb = -(-ctx // bs)
    c = cache[table[:nb].long()].reshape(nb * bs, R)[:ctx].float()
    s = torch.einsum("hnr,jr->hnj", qa.float(), c) * scale
    n = qa.shape[1]
    vis = torch.arange(ctx)[None, :] <= (pos0 + torch.arange(n))[:, None]
    s = s.masked_fill(~vis[None], float("-inf"))
    out.copy_(torch.einsum("hnj,jr->hnr", torch.softmax(s, -1), c))


def latent_attention(qa: torch.Tensor, cache: torch.Tensor, rag: Ragged, scale: float, out: torch.Tensor,
                     workspace=None, part_len: int = 0, impl: int = 0):
    """Causal softmax attention of absorbed queries qa [H, T, R] over the paged latents (keys = values = latents,
    shared by the heads); out [H, T, R] in qa's dtype (fp32 or bf16, the cache's too). Decode rows split their
    context into partitions of `part_len` keys (0: one) merged through `workspace` = (fp32 [rows, 2], fp32 [rows, R])
    with rows >= n_dec * H * partitions. bf16 tensors whose rank is a multiple of 8 run on the matrix cores
    (impl 0); impl 1 keeps them on the fp32 VALU kernel that serves fp32 tensors and odd ranks."""
    H, T, R = qa.shape
    if T == 0:
        return out
    nd = rag.n_dec
    if not qa.is_cuda:
        if nd:
            lens, bt = rag.dec_lens.tolist(), rag.dec_bt
            for i in range(nd):
                _latent_attn_ref(qa[:, i:i + 1], cache, bt[i], lens[i], lens[i] - 1, scale, out[:, i:i + 1])
        if rag.n_pf:
            cu, ctx = rag.pf_cu.tolist(), rag.pf_ctx.tolist()
            for k in range(rag.n_pf):
                n = cu[k + 1] - cu[k]
                if n:
                    r0 = nd + cu[k]
                    _latent_attn_ref(qa[:, r0:r0 + n], cache, rag.pf_bt[k], ctx[k], ctx[k] - n, scale, out[:, r0:r0 + n])
        return out
    if qa.dtype != cache.dtype or out.dtype != qa.dtype:
        raise TypeError("latent_attention: queries, cache and output share one dtype")
    if qa.stride(2) != 1 or out.stride(2) != 1:
        raise ValueError("latent_attention: the rank axis must be contiguous")
    if R > 512:
        raise ValueError("latent_attention: rank up to 512")
    bs = cache.shape[1]
    st = N.stream_ptr()
    if nd:
        parts = 1
        if part_len and workspace is not None and rag.dec_max_len > part_len:
            parts = -(-rag.dec_max_len // part_len)
            room = workspace[0].shape[0] // (nd * H)  # partitions the partial-result buffers hold per row
            if parts > room:
                parts = max(1, room)
                part_len = -(-(-(-rag.dec_max_len // parts)) // 32) * 32
        ml, po = (workspace[0], workspace[1]) if parts > 1 else (None, None)
        N.kcall("mxl_latent_attn", qa.data_ptr(), qa.stride(1), qa.stride(0), cache.data_ptr(), _is16(cache), bs, R,
                rag.dec_bt.data_ptr(), rag.dec_bt.stride(0), None, rag.dec_lens.data_ptr(), nd, nd, 0,
                out.data_ptr(), out.stride(1), out.stride(0), float(scale), H, parts, part_len if parts > 1 else 0,
                N.ptr(ml), N.ptr(po), impl, st)
    if rag.n_pf:
        N.kcall("mxl_latent_attn", qa.data_ptr(), qa.stride(1), qa.stride(0), cache.data_ptr(), _is16(cache), bs, R,
                rag.pf_bt.data_ptr(), rag.pf_bt.stride(0), rag.pf_cu.data_ptr(), rag.pf_ctx.data_ptr(), rag.n_pf,
                T - nd, nd, out.data_ptr(), out.stride(1), out.stride(0), float(scale), H, 1, 0, None, None, impl, st)
    return out


def head_gate_pack(ov: torch.Tensor, gate_pre: torch.Tensor, out: torch.Tensor):
    """out[t, h * dv + e] = ov[h, t, e] * sigmoid(gate_pre[t, h]); ov fp32 [H, T, dv], gate_pre fp32 [T, H] (may be a
    column slice), out fp32 or bf16 [T, H * dv]."""
    H, T, dv = ov.shape
    if T == 0:
        return out
    if not ov.is_cuda:
        o = ov.float().permute(1, 0, 2) * torch.sigmoid(gate_pre.float())[:, :, None]
        out.copy_(o.reshape(T, H * dv))
        return out
    N.kcall("mxl_head_gate_pack", ov.data_ptr(), gate_pre.data_ptr(), gate_pre.stride(0), out.data_ptr(),
            out.stride(0), _is16(out), H, T, dv, N.stream_ptr())
    return out
