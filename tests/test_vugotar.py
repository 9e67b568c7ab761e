"""Vugotar (chunk-masked sink attention beside a gated delta rule, state-space layers, dense / expert feed-forwards,
looped layers) on the engine against the plain float64 oracle of tests/oracle_vugotar.py: every mechanism alone, whole
prompts, token-by-token decoding, prompt portions down to two tokens, unequal batches, reuse of freed blocks and state
slots, keys far back / at page borders / just inside and outside a chunk with peaked softmax weights, odd sizes, long
decoding, greedy generation through the scheduler, graph replays, and the trace runner's command line.

Each engine test runs on the CPU plumbing path (fp32) and, marked gpu, on the HIP kernels in fp32 and bf16."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import oracle_vugotar as O
from localai_tfp_amd.engine.engine import EngineConfig, LLMEngine
from localai_tfp_amd.models import vugotar as VU
from localai_tfp_amd.ops import hybrid as HY
from localai_tfp_amd.ops.sampling import SamplingParams
from localai_tfp_amd.tokenizer import ByteTokenizer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVS = ["cpu", GPU]
RUNS = [("cpu", "float32", 2e-4), pytest.param("cuda", "float32", 2e-4, marks=pytest.mark.gpu),
        pytest.param("cuda", "bfloat16", 6e-2, marks=pytest.mark.gpu)]

SHAPES = {
    # two looped layers (attention + delta rule with a dense feed-forward, state-space with experts + shared expert)
    "plain": dict(hidden=64, vocab=97, pattern=("parallel", "mamba2"), mlps=("dense", "moe"), heads=4, kv_heads=2,
                  dim=16, vdim=16, chunk=24, d_heads=2, d_kv_heads=1, d_dim=16, d_vdim=16, m_heads=4, m_vdim=16,
                  m_state=16, m_groups=2, m_norm_groups=2, ff=96, experts=4, top=2, expert_ff=32, shared_ff=32,
                  router_scale=1.5, left_scale=0.6, right_scale=0.9, loop=(0, 2, 2)),
    # sizes that differ from each other: dim != vdim, partial rotation, a chunk smaller than a page and odd, as many
    # key heads as heads, two taps and five taps, a state size that is no power of two, top == experts, no shared
    # expert, a layer without a feed-forward, no loop, a large eps, stacked projections of odd total width
    "odd": dict(hidden=40, vocab=61, pattern=("mamba2", "parallel", "parallel"), mlps=(None, "moe", "dense"), heads=6,
                kv_heads=3, dim=24, vdim=40, chunk=7, rot_dims=8, rot_base=300.0, scale=0.4, d_heads=3, d_kv_heads=3,
                d_dim=20, d_vdim=12, d_conv=2, m_heads=3, m_vdim=24, m_state=40, m_groups=3, m_norm_groups=1, m_conv=5,
                ff=50, experts=5, top=5, expert_ff=17, shared_ff=0, router_scale=0.7, left_scale=1.4, right_scale=0.5,
                eps=1e-3),
    # states wider than a lane keeps alone (96 and 160 numbers per column), value sizes that are no multiple of 64,
    # one expert of many, one key head for all heads, the loop over the last layer only
    "wide": dict(hidden=48, vocab=53, pattern=("parallel", "mamba2"), mlps=("moe", "dense"), heads=4, kv_heads=1,
                 dim=72, vdim=8, chunk=33, d_heads=2, d_kv_heads=2, d_dim=160, d_vdim=80, d_conv=4, m_heads=2,
                 m_vdim=72, m_state=96, m_groups=1, m_norm_groups=3, m_conv=2, ff=64, experts=9, top=1, expert_ff=16,
                 shared_ff=24, loop=(1, 2, 3)),
}


def build(device="cpu", dtype="float32", seed=0, **kw):
    cfg = VU.make_config(**kw)
    get = VU.synthetic_source(cfg, seed)
    model = VU.VugotarModel.load(cfg, get, torch.device(device), getattr(torch, dtype))
    return cfg, {k: get(k) for k in get.names}, model


def engine(model, max_tokens=256, seqs=4, bs=16, native=False, blocks=None):
    ec = EngineConfig(max_num_seqs=seqs, max_batched_tokens=max_tokens, max_model_len=max_tokens, block_size=bs,
                      num_blocks=blocks or (-(-max_tokens // bs) * seqs + 1), use_graphs=False, overlap=False,
                      native_scheduler=native, logits_rows=max_tokens, gemm_autotune=False)
    return LLMEngine(model, ByteTokenizer(model.cfg.vocab), ec)


def oracle(cfg, tensors, tokens):
    return O.forward(cfg.to_json(), tensors, tokens)[0].float()


def close(got, want, tol, rms=False):
    """Largest difference relative to the largest value. With `rms` (bf16 runs of whole models) every row's root mean
    square difference relative to the root mean square of all values, and the worst tenth of the rows is left out: a
    router's near tie may fall the other way once the router's input is rounded to bf16, and that row and the ones
    that read its state then differ by more than rounding."""
    d = got.double().cpu() - want.double()
    if rms:
        e = (d.pow(2).mean(-1).sqrt() / want.double().pow(2).mean().sqrt()).reshape(-1).sort().values
        err = e[:max(1, len(e) - len(e) // 10)].max().item()
    else:
        err = d.abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert err < tol, err


def run_cuts(eng, key, tokens, cuts):
    """Feed `tokens` of one request in portions of the given sizes; all logits, in order."""
    out, at = [], 0
    for n in cuts:
        last = at + n == len(tokens)
        out.append(eng.replay_step([(key, tokens[at:at + n], list(range(n)))], [key] if last else []))
        at += n
    assert at == len(tokens)
    return torch.cat(out)


def toks(n, vocab, seed=0):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


class _FB:
    """The ragged layout of one step, as the ops read it."""

    def __init__(self, n_dec, chunks, positions, state, dev, slots=None, dec_bt=None, dec_lens=None, pf_bt=None,
                 pf_ctx=None):
        i32 = dict(dtype=torch.int32, device=dev)
        self.T = n_dec + sum(chunks)
        self.n_decode = n_dec
        self.pf_cu_q = torch.tensor(np.concatenate([[0], np.cumsum(chunks)]), **i32) if chunks else None
        self.positions = torch.tensor(positions, **i32)
        self.slots = torch.tensor(slots if slots is not None else [-1] * self.T, **i32)
        self.seq_state = torch.tensor(state, **i32)
        self.dec_block_tables = None if dec_bt is None else torch.tensor(dec_bt, **i32)
        self.dec_seq_lens = None if dec_lens is None else torch.tensor(dec_lens, **i32)
        self.pf_block_tables = None if pf_bt is None else torch.tensor(pf_bt, **i32)
        self.pf_ctx_lens = None if pf_ctx is None else torch.tensor(pf_ctx, **i32)
        self.dec_max_len = max(dec_lens) if dec_lens else 0
        self.pf_q_lens_host, self.pf_ctx_lens_host = list(chunks), list(pf_ctx or [])


def steps_of(n, cuts):
    """[(n_dec, chunks, first position)] of one sequence fed in portions; a single token after the start is a decode
    row."""
    out, at = [], 0
    for c in cuts:
        out.append((1, [], at) if c == 1 and at > 0 else (0, [c], at))
        at += c
    assert at == n
    return out


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
def test_offset_norm_and_embedding(dev):
    g = torch.Generator().manual_seed(1)
    M, C, eps = 5, 72, 0.3  # a large eps shows whether it sits inside the root
    x = torch.randn(M, C, generator=g) * 3
    w = 0.2 * torch.randn(C, generator=g)
    want = O.offset_norm(x.double(), w, eps)
    o32 = torch.empty(M, C, device=dev)
    o16 = torch.empty(M, C, device=dev, dtype=torch.bfloat16)
    HY.offset_rmsnorm(x.to(dev), w.to(dev), eps, out32=o32, out16=o16)
    close(o32, want, 1e-5)
    close(o16.float(), want, 1e-2)
    rows = torch.tensor([3, 0, 3], dtype=torch.int32)
    sel = torch.empty(3, C, device=dev)
    HY.offset_rmsnorm(x.to(dev), w.to(dev), eps, out32=sel, rows=rows.to(dev))
    close(sel, want[rows.long()], 1e-5)
    x2, w2 = torch.randn(2, 4500, generator=g), torch.randn(4500, generator=g)  # wider than a block keeps in registers
    o2 = torch.empty(2, 4500, device=dev)
    HY.offset_rmsnorm(x2.to(dev), w2.to(dev), eps, out32=o2)
    close(o2, O.offset_norm(x2.double(), w2, eps), 1e-5)
    table = torch.randn(11, C, generator=g).to(torch.bfloat16)
    ids = torch.tensor([10, 0, 4, 4], dtype=torch.int32)
    e = torch.empty(4, C, device=dev)
    HY.embed_rows(table.to(dev), ids.to(dev), e)
    HY.embed_rows(table.to(dev), ids.to(dev), e, accumulate=True)
    close(e, 2 * table.double()[ids.long()], 1e-6)


def _attention_case(dev, dt, H, G, dk, dv, rot, chunk, n, cuts, bs, scale, plant=()):
    """Append + attend a sequence in portions through shuffled pages; `plant` = [(query position, key position)]:
    the key is made parallel to the query before rotation-free norms, so that one score stands out."""
    g = torch.Generator().manual_seed(7)
    md = getattr(torch, dt)
    q = torch.randn(n, H * dk, generator=g)
    k = torch.randn(n, G * dk, generator=g)
    v = torch.randn(n, G * dv, generator=g)
    for qi, kj in plant:
        for h in range(H):  # every head's query points at key kj of its group
            gg = h // (H // G)
            q[qi, h * dk:(h + 1) * dk] = k[kj, gg * dk:(gg + 1) * dk]
    eps, base = 1e-6, 100.0
    pos = torch.arange(n)
    qd = O.unit_rms(O.rotary_pairs(q.double().reshape(n, H, dk), pos, rot, base) if rot else
                    q.double().reshape(n, H, dk), eps)
    kd = O.unit_rms(O.rotary_pairs(k.double().reshape(n, G, dk), pos, rot, base) if rot else
                    k.double().reshape(n, G, dk), eps)
    want = O.chunk_sink_attention(qd, kd, v.double().reshape(n, G, dv), scale, chunk).reshape(n, H * dv)
    nb = -(-n // bs)
    table = torch.randperm(nb + 3, generator=g)[:nb].tolist()  # pages out of order
    kc = torch.full((nb + 3, bs, G * dk), 7.0, dtype=md, device=dev)  # stale numbers in unused slots
    vc = torch.full((nb + 3, bs, G * dv), -5.0, dtype=md, device=dev)
    wide = torch.cat([torch.randn(n, 3, generator=g), q, k, v], 1).to(dev)  # the projections as column slices
    got = torch.empty(n, H * dv + 5, device=dev, dtype=md)
    part = (torch.empty(H * 8, 2, device=dev), torch.empty(H * 8, dv, device=dev))  # room for eight partitions
    for n_dec, chunks, at in steps_of(n, cuts):
        c = 1 if n_dec else chunks[0]
        rows = list(range(at, at + c))
        slots = [table[p // bs] * bs + p % bs for p in rows]
        fb = _FB(n_dec, chunks, rows, [0], dev, slots, dec_bt=[table] if n_dec else None,
                 dec_lens=[at + 1] if n_dec else None, pf_bt=None if n_dec else [table],
                 pf_ctx=None if n_dec else [at + c])
        qo = torch.empty(c, H * dk, device=dev, dtype=md)
        w = wide[at:at + c]
        HY.rope_norm_append(w[:, 3:3 + H * dk], w[:, 3 + H * dk:3 + (H + G) * dk], w[:, 3 + (H + G) * dk:],
                            fb.positions, H, G, dk, dv, rot, base, True, eps, qo, kc, vc, fb.slots)
        HY.masked_attention(qo, kc, vc, HY.Ragged(fb), H, G, dk, dv, scale, got[at:at + c, 5:], chunk=chunk, sink=True,
                            out_scale=0.5, workspace=part)
    return got[:, 5:].float() * 2, want


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("gemm_rows", [64, 8])
def test_attention_chunk_edges_pages_and_sink(dev, dt, tol, gemm_rows, monkeypatch):
    """Planted keys carry nearly all the weight: the first key of the query's chunk (just inside), the last key of
    the chunk before (just outside: the output must not move towards it), a key across a page border, the query's own
    position; in prompt portions and in rows decoded alone. On the GPU portions of `gemm_rows` rows and more take
    the library-GEMM route, shorter ones and decoded rows the row kernel."""
    monkeypatch.setattr(HY, "GEMM_MIN_ROWS", gemm_rows)
    chunk, bs, n = 40, 16, 150
    plant = [(79, 40), (119, 80), (120, 119), (121, 120), (95, 81), (149, 127), (60, 60), (39, 0), (41, 39)]
    for cuts in ([n], [37, 2, 41, 1, 1, 38, 1, 1, 1, 27], [118] + [1] * 32):
        got, want = _attention_case(dev, dt, 4, 2, 16, 24, 0, chunk, n, cuts, bs, 4.0, plant)
        close(got, want, tol * (4 if dt == "bfloat16" else 1))
    # partial and full rotation, one key head, sizes that are no multiple of eight, a chunk of one page and a bit
    got, want = _attention_case(dev, dt, 3, 1, 12, 5, 6, 19, 70, [33, 2, 1, 1, 30, 3], 16, 0.7)
    close(got, want, tol)
    got, want = _attention_case(dev, dt, 2, 2, 64, 72, 64, 0, 90, [50, 40], 8, 0.3)  # no chunks: plain causal
    close(got, want, tol)
    # head sizes of 64 and 128 (the matrix-core kernel takes bf16 portions of 16 rows and more): four, two and one
    # query heads per key head, dim != vdim, portions that start and end inside 16-row tiles, pages and chunks
    plant = [(79, 40), (119, 80), (120, 119), (121, 120), (95, 81), (149, 127), (60, 60), (39, 0), (41, 39)]
    for H, G, dk, dv, rot, ch in ((4, 2, 64, 64, 0, 40), (8, 2, 128, 128, 0, 40), (2, 2, 64, 128, 0, 40),
                                  (6, 3, 128, 64, 0, 40)):
        got, want = _attention_case(dev, dt, H, G, dk, dv, rot, ch, 150, [37, 2, 41, 1, 17, 22, 1, 29], bs, 0.5, plant)
        close(got, want, tol * (4 if dt == "bfloat16" else 1))
    got, want = _attention_case(dev, dt, 4, 1, 64, 64, 32, 0, 200, [130, 70], 16, 0.2)  # rotated, plain causal
    close(got, want, tol)
    # rows decoded alone behind 260 and more visible keys: their keys are split into partitions and merged
    plant = [(270, 3), (280, 127), (281, 128), (299, 255), (290, 256), (295, 295)]
    got, want = _attention_case(dev, dt, 2, 1, 16, 16, 16, 0, 300, [200, 60] + [1] * 40, 16, 3.0, plant)
    close(got, want, tol * (4 if dt == "bfloat16" else 1))
    got, want = _attention_case(dev, dt, 4, 1, 64, 64, 64, 0, 300, [200, 60] + [1] * 40, 16, 1.0, plant)  # matrix cores
    close(got, want, tol * (4 if dt == "bfloat16" else 1))
    got, want = _attention_case(dev, dt, 6, 2, 128, 64, 0, 0, 300, [259] + [1] * 41, 16, 0.5, plant)
    close(got, want, tol * (4 if dt == "bfloat16" else 1))


@pytest.mark.parametrize("dev", DEVS)
def test_sink_takes_weight_when_all_scores_are_low(dev):
    """With strongly negative scores the sink holds the denominator: outputs shrink towards zero instead of
    averaging the values."""
    g = torch.Generator().manual_seed(3)
    n, dk, dv = 6, 8, 8
    q = torch.randn(n, dk, generator=g)
    got, want = [], []
    for sink in (True, False):
        kc = torch.zeros(2, 8, dk, device=dev)
        vc = torch.zeros(2, 8, dv, device=dev)
        k, v = -q.clone(), torch.ones(n, dv)
        fb = _FB(0, [n], list(range(n)), [0], dev, list(range(n)), pf_bt=[[0, 1]], pf_ctx=[n])
        qo = torch.empty(n, dk, device=dev)
        HY.rope_norm_append(q.to(dev), k.to(dev), v.to(dev), fb.positions, 1, 1, dk, dv, 0, 10.0, True, 1e-6, qo, kc,
                            vc, fb.slots)
        o = torch.empty(n, dv, device=dev)
        HY.masked_attention(qo, kc, vc, HY.Ragged(fb), 1, 1, dk, dv, 3.0, o, sink=sink)
        got.append(o.cpu())
    assert got[0][0].abs().max() < 1e-6 and torch.allclose(got[1][0], torch.ones(dv), atol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("taps,bias", [(1, False), (2, True), (4, True), (5, False)])
def test_causal_conv_carries_its_tails(dev, taps, bias):
    g = torch.Generator().manual_seed(taps)
    C, n = 70, 41
    x = torch.randn(n, C + 4, generator=g)
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g) if bias else None
    want = O.silu(O.causal_taps(x[:, 4:].double(), w, b))
    tails = torch.full((3, max(1, taps - 1), C), 9.0, device=dev)  # slot 2 holds another sequence's leftovers
    out = torch.empty(n, C, device=dev)
    for n_dec, chunks, at in steps_of(n, [2, 1, 1, 7, 2, 2, 1, 20, 3, 2]):  # portions shorter than the taps
        c = 1 if n_dec else chunks[0]
        fb = _FB(n_dec, chunks, list(range(at, at + c)), [2], dev)
        HY.causal_conv(x.to(dev)[at:at + c, 4:], w.to(dev), b.to(dev) if bias else None, tails, HY.Ragged(fb),
                       out[at:at + c], silu=True)
    close(out, want, 1e-5)
    # two sequences in one step: a decode row beside a fresh prompt chunk that reuses a dirty slot
    tails2 = torch.full((3, max(1, taps - 1), C), -3.0, device=dev)
    first = torch.empty(5, C, device=dev)
    HY.causal_conv(x.to(dev)[:5, 4:], w.to(dev), b.to(dev) if bias else None, tails2,
                   HY.Ragged(_FB(0, [5], list(range(5)), [1], dev)), first, silu=True)
    both = torch.empty(1 + 6, C, device=dev)
    xin = torch.cat([x[5:6, 4:], x[:6, 4:]], 0).to(dev)
    HY.causal_conv(xin, w.to(dev), b.to(dev) if bias else None, tails2,
                   HY.Ragged(_FB(1, [6], [5] + list(range(6)), [1, 0], dev)), both, silu=True)
    close(both[0], want[5], 1e-5)
    close(both[1:], want[:6], 1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("delta,H,G,N,P", [(True, 2, 1, 16, 16), (True, 3, 3, 20, 12), (True, 2, 2, 160, 80),
                                           (False, 4, 2, 16, 8), (False, 3, 1, 40, 24), (False, 2, 1, 96, 72),
                                           (True, 1, 1, 128, 128)])
def test_state_scan_in_portions(dev, delta, H, G, N, P):
    g = torch.Generator().manual_seed(N + P)
    n = 37
    k = torch.randn(n, G * N, generator=g) * (N ** -0.5 if delta else 1.0)
    q = torch.randn(n, G * N, generator=g)
    v = torch.randn(n, H * P, generator=g)
    a_raw, b_raw = torch.randn(n, H, generator=g), torch.randn(n, H, generator=g)
    A_log, dtb = torch.randn(H, generator=g) * 0.3, torch.randn(H, generator=g)
    skip = None if delta else torch.randn(H, generator=g)
    s = O.softplus(a_raw.double() + dtb.double())
    decay = torch.exp(-torch.exp(A_log.double()) * s)
    coef = torch.sigmoid(b_raw.double()) if delta else s
    want = torch.zeros(n, H, P, dtype=torch.float64)
    for h in range(H):
        kk, qq = k.double().reshape(n, G, N)[:, h // (H // G)], q.double().reshape(n, G, N)[:, h // (H // G)]
        vv = v.double().reshape(n, H, P)[:, h]
        if delta:
            want[:, h] = O.delta_rule(qq, kk, vv, coef[:, h], decay[:, h])
        else:
            S = torch.zeros(N, P, dtype=torch.float64)
            for t in range(n):
                S = decay[t, h] * S + coef[t, h] * torch.outer(kk[t], vv[t])
                want[t, h] = S.T @ qq[t] + skip[h].double() * vv[t]
    state = torch.full((2, H, P, N), 4.0, device=dev)  # slot 1 is dirty: position 0 must not read it
    out = torch.empty(n, H * P, device=dev)
    dec, cf = torch.empty(n, H, device=dev), torch.empty(n, H, device=dev)
    HY.scan_coefs(a_raw.to(dev), b_raw.to(dev) if delta else None, A_log.to(dev), dtb.to(dev), dec, cf)
    close(dec, decay, 1e-5)
    close(cf, coef, 1e-5)
    for n_dec, chunks, at in steps_of(n, [9, 1, 2, 1, 1, 20, 3]):
        c = 1 if n_dec else chunks[0]
        fb = _FB(n_dec, chunks, list(range(at, at + c)), [1], dev)
        sl = slice(at, at + c)
        HY.state_scan(k.to(dev)[sl], q.to(dev)[sl], v.to(dev)[sl], dec[sl], cf[sl], None if delta else skip.to(dev),
                      state, HY.Ragged(fb), out[sl], H, G, N, P, delta)
    close(out, want.reshape(n, H * P), 2e-5)
    assert float(state[0].min()) == 4.0  # the other slot is untouched


@pytest.mark.parametrize("dev", DEVS)
def test_unit_heads_group_norm_glu_and_router(dev):
    g = torch.Generator().manual_seed(5)
    T = 6
    x = torch.randn(T, 3 + 4 * 10, generator=g)
    xd = x.clone().to(dev)
    HY.unit_norm_heads(xd[:, 3:], 4, 10, 1e-6, 10 ** -0.5)
    v = x[:, 3:].double().reshape(T, 4, 10)
    close(xd[:, 3:], (v / torch.sqrt((v * v).sum(-1, keepdim=True) + 1e-6) * 10 ** -0.5).reshape(T, 40), 1e-5)
    assert torch.equal(xd[:, :3].cpu(), x[:, :3])
    xd = x.clone().to(dev)  # queries and keys side by side: the first three heads scaled, the last one not
    HY.unit_norm_heads(xd[:, 3:], 4, 10, 1e-6, 0.25, split=3, scale2=1.0)
    sc = torch.tensor([0.25, 0.25, 0.25, 1.0], dtype=torch.float64)[None, :, None]
    close(xd[:, 3:], (v / torch.sqrt((v * v).sum(-1, keepdim=True) + 1e-6) * sc).reshape(T, 40), 1e-5)
    # group norm: gate before the norm over 3 groups with a full-width weight; gate after it with a per-head weight
    y, gt = torch.randn(T, 36, generator=g), torch.randn(T, 36 + 2, generator=g)
    w_full, w_head = torch.randn(36, generator=g), torch.randn(12, generator=g)
    eps = 0.2
    z = y.double() * O.silu(gt[:, 2:].double())
    want = O.unit_rms(z.reshape(T, 3, 12), eps).reshape(T, 36) * w_full.double()
    o = torch.empty(T, 40, device=dev, dtype=torch.bfloat16 if dev == "cuda" else torch.float32)
    HY.gated_group_norm(y.to(dev), gt.to(dev)[:, 2:], w_full.to(dev), eps, 12, o[:, 4:], gate_first=True)
    close(o[:, 4:].float(), want, 1e-2 if dev == "cuda" else 1e-5)
    want = O.unit_rms(y.double().reshape(T, 3, 12), eps).reshape(T, 36) * w_head.double().repeat(3) \
        * O.silu(gt[:, 2:].double()) * 0.9
    o = torch.empty(T, 36, device=dev)
    HY.gated_group_norm(y.to(dev), gt.to(dev)[:, 2:], w_head.to(dev), eps, 12, o, gate_first=False, out_scale=0.9)
    close(o, want, 1e-5)
    # glu with biases; with per-group factors; with a sigmoid factor
    a, b = torch.randn(T, 30, generator=g), torch.randn(T, 30, generator=g)
    ba, bb = torch.randn(30, generator=g), torch.randn(30, generator=g)
    o = torch.empty(T, 30, device=dev)
    HY.glu(a.to(dev), b.to(dev), ba.to(dev), bb.to(dev), o)
    close(o, O.silu(a.double() + ba.double()) * (b.double() + bb.double()), 1e-5)
    fac = torch.randn(T, 5, generator=g)
    fac[0, 2] = 0.0
    HY.glu(a.to(dev), b.to(dev), None, None, o, scale=fac.to(dev), group=6)
    close(o, O.silu(a.double()) * b.double() * fac.double().repeat_interleave(6, 1), 1e-5)
    HY.glu(a.to(dev), b.to(dev), None, None, o, scale=fac.to(dev)[:, 1:2], group=30, scale_sigmoid=True)
    close(o, O.silu(a.double()) * b.double() * torch.sigmoid(fac.double()[:, 1:2]), 1e-5)
    # router: softmax over all, the top ones renormalised and scaled; top == experts; one expert of many
    for E, top in ((7, 3), (5, 5), (70, 1), (130, 4)):
        z = torch.randn(T, E + 1, generator=g) * 2
        wts = torch.empty(T, E, device=dev)
        HY.moe_route(z.to(dev)[:, 1:], top, 1.5, wts, 1e-20)
        s = torch.softmax(z[:, 1:].double(), -1)
        tv, ti = torch.topk(s, top, -1)
        want = torch.zeros(T, E, dtype=torch.float64).scatter_(1, ti, tv / (tv.sum(-1, keepdim=True) + 1e-20) * 1.5)
        close(wts, want, 1e-5)


# ------------------------------------------------------------------------------------------------ whole model
@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_portions_and_decoding(dev, dt, tol, shape):
    """The whole prompt in one step, token-by-token decoding after a prefix, and portions of several sizes down to
    two tokens (cut inside pages, chunks and convolution windows): all give the oracle's logits."""
    cfg, tensors, model = build(dev, dt, seed=3, **SHAPES[shape])
    t = toks(75, cfg.vocab, 5)
    want = oracle(cfg, tensors, t)
    eng = engine(model, 96)
    b16 = dt == "bfloat16"
    tol = tol / 2 if b16 else tol
    close(run_cuts(eng, "whole", t, [75]), want, tol, b16)
    close(run_cuts(eng, "decode", t, [40] + [1] * 35), want, tol, b16)
    close(run_cuts(eng, "cuts", t, [3, 2, 19, 2, 1, 1, 30, 2, 7, 1, 1, 1, 5]), want, tol, b16)
    close(run_cuts(eng, "first", t[:9], [1] * 9), want[:9], tol, b16)  # the first tokens, one by one from position 0
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 4


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_recurrent_layers_only(dev, dt, tol):
    """A model without any attention layer: the paged pool is empty, blocks are bookkeeping only (the engine sizes
    them without a pool), states and tails carry everything."""
    kw = dict(SHAPES["plain"], pattern=("mamba2", "mamba2", "mamba2"), mlps=("dense", None, "moe"), loop=(1, 3, 2))
    cfg, tensors, model = build(dev, dt, seed=13, **kw)
    assert model.cache_ranks() == []
    t = toks(60, cfg.vocab, 3)
    want = oracle(cfg, tensors, t)
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=64, max_model_len=64, block_size=16, use_graphs=False,
                      overlap=False, native_scheduler=False, logits_rows=64, gemm_autotune=False)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
    assert eng.bm.num_blocks == 2 * 4 + 1
    b16 = dt == "bfloat16"
    close(run_cuts(eng, "a", t, [60]), want, tol / 2 if b16 else tol, b16)
    close(run_cuts(eng, "b", t, [7, 2, 30] + [1] * 21), want, tol / 2 if b16 else tol, b16)


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_residual_after_every_layer_run(dev, dt, tol):
    """The residual stream after each run of a layer (a looped layer counts every pass)."""
    cfg, tensors, model = build(dev, dt, seed=9, **SHAPES["plain"])
    t = toks(30, cfg.vocab, 2)
    _, layers = O.forward(cfg.to_json(), tensors, t)
    assert layers.shape[0] == 4  # two layers, looped twice
    eng = engine(model, 32)
    for r in range(1, layers.shape[0] + 1):
        orig = eng._build_fb  # the engine's own planner builds the step; stop_layer cuts the forward short

        def fb_cut(plan, tt=None, _r=r):
            fb = orig(plan, tt)
            fb.stop_layer = _r
            return fb
        eng._build_fb = fb_cut
        try:
            eng.replay_step([("k%d" % r, t, [0])], ["k%d" % r])
        finally:
            eng._build_fb = orig
        close(eng.ws.x[:len(t)].float(), layers[r - 1].float(), tol, dt == "bfloat16")


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_unequal_batches_reuse_blocks_and_slots(dev, dt, tol):
    """Five requests of unequal length through an engine with three state slots and a pool smaller than their sum:
    portions of some beside single tokens of others; finished requests hand their blocks and slot to new ones. Every
    request's logits equal those it gets alone."""
    cfg, tensors, model = build(dev, dt, seed=11, **SHAPES["plain"])
    reqs = {k: toks(n, cfg.vocab, 40 + n) for k, n in (("a", 61), ("b", 9), ("c", 33), ("d", 50), ("e", 2))}
    want = {k: oracle(cfg, tensors, v) for k, v in reqs.items()}
    eng = engine(model, max_tokens=160, seqs=3, blocks=11)  # 10 usable pages of 16 tokens
    plan = [[("a", 17), ("b", 2)], [("a", 2), ("b", 1), ("c", 30)], [("a", 1), ("b", 1), ("c", 1)],
            [("a", 30), ("b", 5), ("c", 2)], [("a", 11), ("d", 20)], [("d", 1), ("e", 2)], [("d", 29)]]
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            tk = reqs[k][at[k]:at[k] + n]
            entries.append((k, tk, list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = eng.replay_step(entries, end)
        r = 0
        for k, tk, _ in entries:
            got[k].append(out[r:r + len(tk)])
            r += len(tk)
    for k in reqs:
        assert at[k] == len(reqs[k])
        close(torch.cat(got[k]), want[k], tol / 2 if dt == "bfloat16" else tol, dt == "bfloat16")
        # and the same request alone, in the same number format: no router tie falls differently here
        alone = run_cuts(eng, "alone-" + k, reqs[k], [len(reqs[k])])
        close(torch.cat(got[k]), alone, 2e-4 if dt == "float32" else 4e-3)
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 3


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_peaked_attention_far_keys_and_long_decode(dev, dt, tol):
    """A large score scale makes single keys dominate, so a lost or shifted key anywhere in a long chunk (page
    borders, the chunk's first key) moves the logits; then 70 tokens decoded one by one across two chunk edges."""
    kw = dict(SHAPES["plain"], scale=2.5, chunk=96, loop=(0, 0, 1))
    cfg, tensors, model = build(dev, dt, seed=21, **kw)
    t = toks(260, cfg.vocab, 8)
    want = oracle(cfg, tensors, t)
    eng = engine(model, max_tokens=272, seqs=2)
    got = run_cuts(eng, "x", t, [187, 3] + [1] * 70)
    close(got, want, tol * 2, rms=dt == "bfloat16")


# ------------------------------------------------------------------------------------------------ serving path
@pytest.mark.parametrize("dev,dt", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("native", [False, True])
def test_greedy_generation_through_the_scheduler(dev, dt, native):
    """engine.submit: chunked prefill, continuous batching of three requests, greedy sampling; each request's tokens
    equal the oracle's greedy continuation."""
    cfg, tensors, model = build(dev, dt, seed=4, **SHAPES["plain"])
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=24, prefill_chunk=10, max_model_len=128, block_size=16,
                      num_blocks=20, use_graphs=False, native_scheduler=native, gemm_autotune=False)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
    if native and not eng.native_sched:
        pytest.skip("native runtime not built")
    prompts = [toks(n, cfg.vocab, 30 + n) for n in (27, 5, 13)]
    from localai_tfp_amd.engine.sequence import Request
    hs = [eng.submit(Request(p, SamplingParams(temperature=0.0, ignore_eos=True), 12)) for p in prompts]
    eng.run_until_done()
    for p, h in zip(prompts, hs):
        ids = [i for o in h for i in o.token_ids]
        seq = list(p)
        for _ in range(12):
            seq.append(int(oracle(cfg, tensors, seq)[-1].argmax()))
        assert ids == seq[len(p):]
    assert len(eng.state_slots.owner) <= 2


@pytest.mark.gpu
def test_decode_graphs_replay_like_the_oracle():
    """Decode-only steps replay captured graphs (several buckets as requests come and go, eager prompt chunks
    between the replays); every request still yields the oracle's greedy tokens, also after slots were reused."""
    cfg, tensors, model = build("cuda", "float32", seed=4, **SHAPES["odd"])
    ec = EngineConfig(max_num_seqs=3, max_batched_tokens=32, prefill_chunk=9, max_model_len=128, block_size=16,
                      num_blocks=24, use_graphs=True, gemm_autotune=False)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
    from localai_tfp_amd.engine.sequence import Request
    prompts = [toks(n, cfg.vocab, 70 + n) for n in (21, 4, 30, 11, 17)]
    gens = [14, 25, 6, 9, 12]
    hs = [eng.submit(Request(p, SamplingParams(temperature=0.0, ignore_eos=True), g)) for p, g in zip(prompts, gens)]
    eng.run_until_done()
    assert eng.stats["graph_steps"] >= 5
    for p, g, h in zip(prompts, gens, hs):
        ids = [i for o in h for i in o.token_ids]
        seq = list(p)
        for _ in range(g):
            seq.append(int(oracle(cfg, tensors, seq)[-1].argmax()))
        assert ids == seq[len(p):]


@pytest.mark.parametrize("native", [False, True])
def test_preempted_request_recomputes_its_state(native):
    """A pool too small for both requests' growth: one is preempted, loses its blocks and state slot, and is
    recomputed from position 0 later; both still produce the oracle's greedy tokens."""
    cfg, tensors, model = build("cpu", "float32", seed=8, **SHAPES["plain"])
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=64, max_model_len=128, block_size=16, num_blocks=8,
                      use_graphs=False, native_scheduler=native, gemm_autotune=False)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
    if native and not eng.native_sched:
        pytest.skip("native runtime not built")
    from localai_tfp_amd.engine.sequence import Request
    prompts = [toks(30, cfg.vocab, 51), toks(28, cfg.vocab, 52)]
    hs = [eng.submit(Request(p, SamplingParams(temperature=0.0, ignore_eos=True), 40)) for p in prompts]
    eng.run_until_done()
    assert eng.stats["preemptions"] > 0
    for p, h in zip(prompts, hs):
        ids = [i for o in h for i in o.token_ids]
        seq = list(p)
        for _ in range(40):
            seq.append(int(oracle(cfg, tensors, seq)[-1].argmax()))
        assert ids == seq[len(p):]


def test_config_reader_and_checkpoint_round_trip(tmp_path):
    cfg = VU.make_config(**SHAPES["odd"])
    get = VU.synthetic_source(cfg, 1)
    VU.save_checkpoint(cfg, get, str(tmp_path))
    assert VU.is_vugotar_dir(str(tmp_path))
    cfg2, get2 = VU.dir_source(str(tmp_path))
    assert cfg2.to_json() == cfg.to_json() and cfg2.layers[0].mlp is None and cfg2.layers[1].mlp.shared_ff is None
    assert torch.equal(get2("l1.mix.left.q"), get("l1.mix.left.q")) and get2("l0.mlp.gate") is None
    assert [i for i, _ in VU.make_config(**SHAPES["wide"]).runs()] == [0, 1, 1, 1]
    assert VU.make_config(**SHAPES["plain"]).runs() == [(0, False), (1, False), (0, True), (1, False)]
    from localai_tfp_amd.models.loader import load_llm
    m, _tok, c, _ = load_llm(str(tmp_path), "cpu")
    assert isinstance(m, VU.VugotarModel) and c.layers[1].mixer.left.chunk == 7
    for path, val in ((("layers", 0, "type"), "something_else"), (("layers", 1, "mlp", "kind"), "sparse")):
        bad = cfg.to_json()
        node = bad
        for p in path[:-1]:
            node = node[p]
        node[path[-1]] = val
        with pytest.raises(ValueError):
            VU.VugotarConfig.from_json(bad)
    tensors = {k: get(k) for k in get.names}
    tensors["l1.mix.left.q"] = tensors["l1.mix.left.q"][:-1]
    with pytest.raises(ValueError):
        VU.VugotarModel.load(cfg, tensors.get, "cpu")


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run on a checkpoint directory: steps on stdin, one logits file per step that wants any."""
    cfg = VU.make_config(**SHAPES["plain"])
    get = VU.synthetic_source(cfg, 6)
    mdir, odir = str(tmp_path / "m"), str(tmp_path / "o")
    VU.save_checkpoint(cfg, get, mdir)
    a, b = toks(21, cfg.vocab, 1), toks(9, cfg.vocab, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:12], "want": [0, 11]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[12:13], "want": []}, {"id": "b", "tokens": b, "want": [8]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:], "want": [7, 0]}], "end": ["a"]}]
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", mdir, "--dtype", "float32", "--out", odir,
                        "--max-tokens", "128", "--device", "cpu"], input="".join(json.dumps(s) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    tensors = {k: get(k) for k in get.names}
    wa, wb = oracle(cfg, tensors, a), oracle(cfg, tensors, b)
    rd = lambda n: torch.from_numpy(np.fromfile(os.path.join(odir, "%d.f32" % n), dtype="<f4").reshape(-1, cfg.vocab))  # noqa: E731
    close(rd(0), wa[[0, 11]], 2e-4)
    close(rd(1), wb[[8]], 2e-4)
    close(rd(2), wa[[20, 13]], 2e-4)


def test_served_through_the_llm_worker(tmp_path):
    """The gRPC LLM worker loads a Vugotar checkpoint directory like any other model and streams a completion whose
    tokens are the oracle's greedy continuation (byte-level tokenizer: one token per prompt byte after BOS)."""
    from localai_tfp_amd.grpc import pb
    from localai_tfp_amd.grpc.client import BackendClient
    from localai_tfp_amd.grpc.server import AioServer
    from localai_tfp_amd.workers.llm import LLMServicer
    cfg = VU.make_config(**dict(SHAPES["plain"], vocab=300))
    get = VU.synthetic_source(cfg, 12)
    VU.save_checkpoint(cfg, get, str(tmp_path))
    svc = LLMServicer(device="cpu")
    server = AioServer(svc, "127.0.0.1:0", max_workers=4)
    c = BackendClient(f"127.0.0.1:{server.port}")
    try:
        r = c.load_model(pb.ModelOptions(Model=str(tmp_path), ContextSize=256))
        assert r.success, r.message
        assert isinstance(svc.engine.model, VU.VugotarModel)
        o = pb.PredictOptions(Prompt="hybrid", Tokens=6, Temperature=0.0, IgnoreEOS=True)
        a = c.predict(o)
        chunks = list(c.predict_stream(o))
        assert a.tokens == 6 and b"".join(x.message for x in chunks) == a.message
        tok = svc.engine.tok
        seq = list(tok.encode("hybrid"))
        assert a.prompt_tokens == len(seq)
        tensors = {k: get(k) for k in get.names}
        want = []
        for _ in range(6):
            want.append(int(oracle(cfg, tensors, seq + want)[-1].argmax()))
        assert tok.decode(want).encode(errors="replace") == a.message or a.message == tok.decode(want).encode()
    finally:
        c.close()
        if svc.engine is not None:
            svc.engine.shutdown()
        server.stop()
