"""Vugotar: a hybrid decoder. Every layer reads ONE offset RMS norm of the fp32 residual and adds the sum of a mixer
and a feed-forward that both read it:

    h  = x / rms(x) * (1 + w)
    x += mixer(h) + ff(h)

Mixers (`type`):
  parallel  two mixers side by side, left_scale * left(h) + right_scale * right(h):
            left   softmax attention with grouped key/value heads, rotary positions on neighbouring pairs of the first
                   rot.dims numbers of each head, a unit-RMS norm of every query and key head after the rotation, a
                   chunked causal mask (a token sees the earlier tokens of its own block of mask.size positions) and
                   a sink term in the softmax denominator;
            right  gated delta rule: short causal convolutions + SiLU on q, k, v, unit-length q and k per head, a
                   per-head decay exp(-exp(A_log) softplus(a + dt_bias)) and write strength sigmoid(b), an fp32 state
                   [dim, vdim] per head, the read-out normed per head and gated by silu(g);
  mamba2    state-space duality form: one input projection laid out z | x | B | C | dt, a causal convolution + SiLU over
            x | B | C, dt = softplus(dt + dt_bias), S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, gated by
            silu(z) and normed in norm_groups parts.
Feed-forwards (`mlp.kind`): dense (SiLU-gated, with biases), moe (softmax router over all experts, the top ones
renormalised and scaled, plus an optional shared expert behind a sigmoid gate), or none.
`loop` runs layers start .. stop-1 `times` times with the same weights; every pass has its own cache and state, and
the embedding output is added to the residual before each pass but the first.

How a layer maps onto launches (T rows of a ragged engine step):

    norm                      -> hin (GEMM operand)                                   hybrid_ops.hip
    y = hin W_in^T            every projection that reads h, stacked into ONE GEMM    hipBLASLt, fp32 out
    left:  rope + head norm + paged append; masked attention -> cat[:, left]          hybrid_ops / hybrid_attn.hip
    right: conv + SiLU (q|k|v stacked); unit norms; decay / beta; scan; head norm * silu(g) -> cat[:, right]
    mamba2: conv + SiLU over x|B|C; decay / dt; scan (+ D x); silu(z) gate + group norm -> cat[:, mixer]
    ff:    glu -> cat[:, ff] (dense: biases; moe: router -> dense [T, E] routing weights, every expert's gate/up
           evaluated from the stacked GEMM and its activation scaled by its routing weight, 0 when not chosen;
           shared expert scaled by its sigmoid gate)
    x += cat W_out^T (+ bias) every output projection (left o, right o, down, shared down, all experts' down
                              stacked along K) as ONE GEMM accumulating into the fp32 residual

The mixer scales are applied to the activations that feed the output GEMM. Evaluating every expert costs
experts / top times the routed arithmetic but keeps the step free of host synchronisation and data-dependent shapes
(it replays as a hipGraph) and reads each expert's weights once per step.

The engine sees `cache_kind = "hybrid"`: paged key / value pools for the attention of every layer run plus one state
slot per live sequence holding recurrent states and convolution tails (engine/kv_cache.py HybridCache, SlotPool).

`dtype` bf16: GEMM operands and the pools are bf16, everything between GEMMs fp32. `dtype` fp32: all fp32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import torch

from ..ops import hybrid as HY
from ..ops.dense import Dense

ARCH = "Vugotar"
DELTA_UNIT_EPS = 1e-6  # inside the root of the delta rule's unit-length q and k
ROUTE_EPS = 1e-20  # added to the sum of the chosen experts' scores


@dataclass
class AttnCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    chunk: int  # 0: plain causal


@dataclass
class DeltaCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass
class ParallelCfg:
    left: AttnCfg
    right: DeltaCfg
    left_scale: float
    right_scale: float


@dataclass
class Mamba2Cfg:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim


@dataclass
class MlpCfg:
    kind: str  # dense | moe
    ff: int  # dense width, or one expert's
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0
    shared_ff: int | None = None


@dataclass
class VugotarLayerCfg:
    type: str  # parallel | mamba2
    mixer: ParallelCfg | Mamba2Cfg
    mlp: MlpCfg | None


def _need(cond: bool, what: str):
    if not cond:
        raise ValueError(f"Vugotar configuration: {what}")


@dataclass
class VugotarConfig:
    name: str = "vugotar"
    arch: str = "vugotar"
    hidden: int = 256
    vocab: int = 512
    layers: list = field(default_factory=list)
    loop: tuple = (0, 0, 1)  # (start, stop, times)
    rms_eps: float = 1e-6
    ctx_train: int = 1 << 20  # rotary angles are computed from the position: the engine's max_model_len is the limit
    extra: dict = field(default_factory=dict)
    # fields the engine / workers read off every model config
    head_dim: int = 1
    n_heads: int = 1
    n_kv_heads: int = 1
    embed_scale: float = 1.0
    tie_embeddings: bool = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """[(layer index, add the embedding output first)] in the order the layers run."""
        n = len(self.layers)
        a, b, k = self.loop
        if k <= 1 or b <= a:
            return [(i, False) for i in range(n)]
        out = [(i, False) for i in range(a)]
        for r in range(k):
            out += [(i, r > 0 and i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    @classmethod
    def from_json(cls, d: dict, name: str = "vugotar") -> "VugotarConfig":
        if d.get("architecture") != ARCH:
            raise ValueError(f"not a {ARCH} configuration")
        layers = []
        for i, e in enumerate(d["layers"]):
            m = e["mixer"]
            if e["type"] == "parallel":
                a, r = m["left"], m["right"]
                rot = a.get("rot") or {}
                left = AttnCfg(int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"]), float(a["scale"]),
                               int(rot.get("dims", 0)), float(rot.get("base", 10000.0)),
                               int((a.get("mask") or {}).get("size", 0)))
                right = DeltaCfg(int(r["heads"]), int(r["kv_heads"]), int(r["dim"]), int(r["vdim"]), int(r["conv"]))
                _need(left.heads % left.kv_heads == 0 and right.heads % right.kv_heads == 0,
                      f"layer {i}: heads are a multiple of kv_heads")
                _need(left.rot_dims % 2 == 0 and left.rot_dims <= left.dim, f"layer {i}: rot.dims even and <= dim")
                mixer = ParallelCfg(left, right, float(m["left_scale"]), float(m["right_scale"]))
            elif e["type"] == "mamba2":
                mixer = Mamba2Cfg(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]),
                                  int(m["norm_groups"]), int(m["conv"]))
                _need(mixer.heads % mixer.groups == 0 and mixer.inner % mixer.norm_groups == 0,
                      f"layer {i}: heads / groups and inner / norm_groups are whole")
            else:
                raise ValueError(f"layer {i}: unknown mixer {e['type']!r}")
            f = e.get("mlp")
            if f is None:
                mlp = None
            elif f.get("kind") == "dense":
                mlp = MlpCfg("dense", int(f["ff"]))
            elif f.get("kind") == "moe":
                r = f["router"]
                sh = f.get("shared")
                mlp = MlpCfg("moe", int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]),
                             float(r.get("scale", 1.0)), int(sh["ff"]) if sh else None)
                _need(0 < mlp.top <= mlp.experts, f"layer {i}: 1 <= top <= experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward {f.get('kind')!r}")
            layers.append(VugotarLayerCfg(e["type"], mixer, mlp))
        lp = d.get("loop") or {}
        loop = (int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1)))
        _need(0 <= loop[0] <= loop[1] <= len(layers), "loop: 0 <= start <= stop <= layers")
        return cls(name=name, hidden=int(d["width"]), vocab=int(d["vocab"]), layers=layers, loop=loop,
                   rms_eps=float(d["norm"]["eps"]))

    def to_json(self) -> dict:
        ls = []
        for L in self.layers:
            m = L.mixer
            if L.type == "parallel":
                a, r = m.left, m.right
                left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                        "rot": {"dims": a.rot_dims, "base": a.rot_base}}
                if a.chunk:
                    left["mask"] = {"size": a.chunk}
                mj = {"left": left, "left_scale": m.left_scale, "right_scale": m.right_scale,
                      "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim, "conv": r.conv}}
            else:
                mj = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups,
                      "norm_groups": m.norm_groups, "conv": m.conv}
            f = L.mlp
            if f is None:
                fj = None
            elif f.kind == "dense":
                fj = {"kind": "dense", "ff": f.ff}
            else:
                fj = {"kind": "moe", "expert": {"ff": f.ff},
                      "router": {"experts": f.experts, "top": f.top, "scale": f.router_scale}}
                if f.shared_ff:
                    fj["shared"] = {"ff": f.shared_ff}
            ls.append({"type": L.type, "mixer": mj, "mlp": fj})
        return {"architecture": ARCH, "width": self.hidden, "vocab": self.vocab, "norm": {"eps": self.rms_eps},
                "loop": {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}, "layers": ls}


def make_config(hidden=256, vocab=512, pattern=("parallel", "mamba2"), heads=4, kv_heads=2, dim=32, vdim=32, chunk=64,
                rot_dims=None, rot_base=10000.0, scale=None, d_heads=2, d_kv_heads=1, d_dim=32, d_vdim=32, d_conv=3,
                m_heads=4, m_vdim=32, m_state=16, m_groups=1, m_norm_groups=1, m_conv=4, ff=512, mlps=("dense",),
                experts=4, top=2, expert_ff=128, shared_ff=128, router_scale=1.0, left_scale=1.0, right_scale=1.0,
                loop=(0, 0, 1), eps=1e-6, name="vugotar") -> VugotarConfig:
    """A configuration whose i-th layer has mixer pattern[i] and feed-forward mlps[i % len(mlps)]
    ("dense" | "moe" | None)."""
    layers = []
    for i, t in enumerate(pattern):
        if t == "parallel":
            mixer = ParallelCfg(AttnCfg(heads, kv_heads, dim, vdim, float(scale if scale is not None else dim ** -0.5),
                                        dim if rot_dims is None else rot_dims, rot_base, chunk),
                                DeltaCfg(d_heads, d_kv_heads, d_dim, d_vdim, d_conv), left_scale, right_scale)
        else:
            mixer = Mamba2Cfg(m_heads, m_vdim, m_state, m_groups, m_norm_groups, m_conv)
        k = mlps[i % len(mlps)]
        mlp = None if k is None else MlpCfg("dense", ff) if k == "dense" else \
            MlpCfg("moe", expert_ff, experts, top, router_scale, shared_ff or None)
        layers.append(VugotarLayerCfg(t, mixer, mlp))
    return VugotarConfig(name=name, hidden=hidden, vocab=vocab, layers=layers, loop=tuple(loop), rms_eps=eps)


# sizes of the order of a 1B / 7B decoder (bench / synthetic checkpoints): attention + delta-rule layers with dense and
# expert feed-forwards, every fourth layer a state-space layer
SYNTHETIC = {
    "vugotar-tiny": dict(hidden=256, vocab=512, pattern=("parallel", "mamba2", "parallel"), mlps=("dense", "moe")),
    "vugotar-1b": dict(hidden=2048, vocab=32000, pattern=("parallel", "parallel", "parallel", "mamba2") * 4, heads=16,
                       kv_heads=4, dim=128, vdim=128, chunk=2048, d_heads=8, d_kv_heads=4, d_dim=128, d_vdim=128,
                       m_heads=32, m_vdim=64, m_state=128, m_groups=1, ff=8192, mlps=("dense",)),
    "vugotar-7b": dict(hidden=4096, vocab=32000, pattern=("parallel", "parallel", "parallel", "mamba2") * 8, heads=32,
                       kv_heads=8, dim=128, vdim=128, chunk=2048, d_heads=16, d_kv_heads=8, d_dim=128, d_vdim=128,
                       m_heads=64, m_vdim=64, m_state=128, m_groups=1, ff=14336, mlps=("dense",)),
}


@dataclass
class VugotarWeights:
    """Device tensors of one layer, with the column layout of its two stacked GEMMs."""
    norm: torch.Tensor
    w_in: Dense
    w_out: Dense
    cols: dict  # name -> first column of the projection in the input GEMM's output
    n_in: int
    k_out: int
    conv_w: torch.Tensor  # [channels, taps] fp32 (q|k|v of the delta rule, or x|B|C)
    conv_b: torch.Tensor | None
    A_log: torch.Tensor
    dt_bias: torch.Tensor
    mix_norm: torch.Tensor
    skip: torch.Tensor | None  # D of the state-space layer
    gate_b: torch.Tensor | None
    up_b: torch.Tensor | None


class VugotarWorkspace:
    """Step scratch sized for the largest step; forward() only takes views (static addresses for graph capture)."""

    def __init__(self, model: "VugotarModel", max_tokens: int, max_seqs: int, logits_rows: int, max_parts: int = 16):
        cfg, dev, md = model.cfg, model.device, model.dtype
        T, C = max_tokens, cfg.hidden
        f32 = dict(dtype=torch.float32, device=dev)
        m16 = dict(dtype=md, device=dev)
        self.max_tokens, self.max_seqs = T, max_seqs
        self.logits_rows = S = max(max_seqs, logits_rows)
        Ws = list(model.weights.values())
        n_in = max(W.n_in for W in Ws)
        k_out = max(W.k_out for W in Ws)
        n_conv = max(W.conv_w.shape[0] for W in Ws)
        n_heads = max(W.A_log.numel() for W in Ws)
        n_scan, n_q, n_e = 1, 1, 1
        for L in cfg.layers:
            m = L.mixer
            if L.type == "parallel":
                n_scan = max(n_scan, m.right.heads * m.right.vdim)
                n_q = max(n_q, m.left.heads * m.left.dim)
            else:
                n_scan = max(n_scan, m.inner)
            if L.mlp is not None and L.mlp.kind == "moe":
                n_e = max(n_e, L.mlp.experts)
        self.x = torch.empty((T, C), **f32)
        self.hin = torch.empty((T, C), **m16)
        self.y = torch.empty((T * n_in,), **f32)
        self.conv = torch.empty((T * n_conv,), **f32)
        self.decay = torch.empty((T * n_heads,), **f32)
        self.coef = torch.empty((T * n_heads,), **f32)
        self.scan = torch.empty((T * n_scan,), **f32)
        self.q = torch.empty((T * n_q,), **m16)
        self.cat = torch.zeros((T * k_out,), **m16)  # zero: padded columns are read, never written
        self.route = torch.empty((T * n_e,), **f32)
        self.hs = torch.empty((S, C), **m16)
        self.logits = torch.empty((S, cfg.vocab), **f32)
        # partial results of decode rows whose visible keys are split into partitions
        h_att = max([L.mixer.left.heads for L in cfg.layers if L.type == "parallel"] or [1])
        v_att = max([L.mixer.left.vdim for L in cfg.layers if L.type == "parallel"] or [1])
        rows = HY.DECODE_WAVES + max_seqs * h_att  # few sequences take many partitions each, many take few
        self.part_ml = torch.empty((rows, 2), **f32)
        self.part_o = torch.empty((rows, v_att), **f32)


class VugotarModel:
    cache_kind = "hybrid"
    tp_size = 1
    n_kv = 1
    n_heads = 1

    def __init__(self, cfg: VugotarConfig, device="cpu", dtype=None):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype is None:
            dtype = torch.bfloat16 if self.device.type == "cuda" else torch.float32
        if self.device.type != "cuda":
            dtype = torch.float32  # the CPU plumbing path runs everything in fp32
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Vugotar runs in bfloat16 or float32")
        self.dtype = dtype
        self.weights: dict[int, VugotarWeights] = {}
        self.embed: torch.Tensor | None = None
        self.final_norm = None
        self.head: Dense | None = None
        self.last_hidden = None
        self.runs = cfg.runs()

    # ------------------------------------------------------------------ engine hooks
    def cache_spec(self) -> list:
        spec = []
        for li, _ in self.runs:
            L = self.cfg.layers[li]
            m = L.mixer
            if L.type == "parallel":
                a, r = m.left, m.right
                spec.append({"kv": (a.kv_heads * a.dim, a.kv_heads * a.vdim), "state": (r.heads, r.vdim, r.dim),
                             "tails": (r.conv - 1, 2 * r.kv_heads * r.dim + r.heads * r.vdim)})
            else:
                spec.append({"state": (m.heads, m.vdim, m.state),
                             "tails": (m.conv - 1, m.inner + 2 * m.groups * m.state)})
        return spec

    def make_cache(self, num_blocks: int, block_size: int, state_slots: int):
        from ..engine.kv_cache import HybridCache
        return HybridCache(self.cache_spec(), num_blocks, block_size, self.device, self.dtype, state_slots)

    def cache_ranks(self):
        """Pool numbers per token of every run with attention (keys + values)."""
        return [sum(e["kv"]) for e in self.cache_spec() if e.get("kv")]

    def make_workspace(self, max_tokens: int, max_seqs: int, logits_rows: int = 0, max_parts: int = 64):
        return VugotarWorkspace(self, max_tokens, max_seqs, logits_rows, max_parts)

    def weight_bytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size() + self.head.w.numel() * self.head.w.element_size()
        for W in self.weights.values():
            n += (W.w_in.w.numel() + W.w_out.w.numel()) * W.w_in.w.element_size()
        return n

    # ------------------------------------------------------------------ loading
    @classmethod
    def load(cls, cfg: VugotarConfig, get, device="cpu", dtype=None) -> "VugotarModel":
        """`get(name)` -> torch tensor (any float dtype) of the checkpoint tensor `name`."""
        m = cls(cfg, device, dtype)
        dev, md = m.device, m.dtype
        C = cfg.hidden

        def t(name, shape):
            a = get(name)
            if a is None:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            if tuple(a.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(a.shape)}, configuration says {tuple(shape)}")
            return a.float()

        def f32(name, shape):
            return t(name, shape).contiguous().to(dev)

        for i, L in enumerate(cfg.layers):
            p, mx = f"l{i}.mix.", L.mixer
            rows, cols, outs, n = [], {}, [], 0

            def add(key, w):
                nonlocal n
                cols[key] = n
                rows.append(w)
                n += w.shape[0]

            skip = conv_b = None
            if L.type == "parallel":
                a, r = mx.left, mx.right
                add("lq", t(p + "left.q", (a.heads * a.dim, C)))
                add("lk", t(p + "left.k", (a.kv_heads * a.dim, C)))
                add("lv", t(p + "left.v", (a.kv_heads * a.vdim, C)))
                add("rq", t(p + "right.q", (r.kv_heads * r.dim, C)))
                add("rk", t(p + "right.k", (r.kv_heads * r.dim, C)))
                add("rv", t(p + "right.v", (r.heads * r.vdim, C)))
                add("rg", t(p + "right.g", (r.heads * r.vdim, C)))
                add("rb", t(p + "right.b", (r.heads, C)))
                add("ra", t(p + "right.a", (r.heads, C)))
                conv_w = torch.cat([t(p + "right.q.conv", (r.kv_heads * r.dim, r.conv)),
                                    t(p + "right.k.conv", (r.kv_heads * r.dim, r.conv)),
                                    t(p + "right.v.conv", (r.heads * r.vdim, r.conv))], 0)
                A_log, dt_bias = f32(p + "right.A_log", (r.heads,)), f32(p + "right.dt_bias", (r.heads,))
                mix_norm = f32(p + "right.norm", (r.vdim,))
                outs += [t(p + "left.o", (C, a.heads * a.vdim)), t(p + "right.o", (C, r.heads * r.vdim))]
            else:
                inner, gn = mx.inner, mx.groups * mx.state
                add("in", t(p + "in", (2 * inner + 2 * gn + mx.heads, C)))
                conv_w = t(p + "conv", (inner + 2 * gn, mx.conv))
                conv_b = f32(p + "conv.b", (inner + 2 * gn,))
                A_log, dt_bias = f32(p + "A_log", (mx.heads,)), f32(p + "dt_bias", (mx.heads,))
                skip = f32(p + "D", (mx.heads,))
                mix_norm = f32(p + "norm", (inner,))
                outs.append(t(p + "o", (C, inner)))
            f, q = L.mlp, f"l{i}.mlp."
            gate_b = up_b = out_b = None
            if f is not None and f.kind == "dense":
                add("gate", t(q + "gate", (f.ff, C)))
                add("up", t(q + "up", (f.ff, C)))
                gate_b, up_b = f32(q + "gate.b", (f.ff,)), f32(q + "up.b", (f.ff,))
                outs.append(t(q + "down", (C, f.ff)))
                out_b = t(q + "down.b", (C,))
            elif f is not None:
                add("router", t(q + "router", (f.experts, C)))
                if f.shared_ff:
                    add("sg", t(q + "shared.sg", (1, C)))
                    add("sgate", t(q + "shared.gate", (f.shared_ff, C)))
                    add("sup", t(q + "shared.up", (f.shared_ff, C)))
                    outs.append(t(q + "shared.down", (C, f.shared_ff)))
                add("egate", torch.cat([t(f"{q}e{e}.gate", (f.ff, C)) for e in range(f.experts)], 0))
                add("eup", torch.cat([t(f"{q}e{e}.up", (f.ff, C)) for e in range(f.experts)], 0))
                outs += [t(f"{q}e{e}.down", (C, f.ff)) for e in range(f.experts)]
            # both stacked GEMMs get whole 16-byte rows: zero rows / columns up to a multiple of 8 (the padded columns
            # of the output GEMM's operand are never written and stay zero)
            w_in, w_out = torch.cat(rows, 0), torch.cat(outs, 1)
            if n % 8:
                w_in = torch.cat([w_in, torch.zeros(8 - n % 8, C)], 0)
                n = w_in.shape[0]
            if w_out.shape[1] % 8:
                w_out = torch.cat([w_out, torch.zeros(C, 8 - w_out.shape[1] % 8)], 1)
            m.weights[i] = VugotarWeights(
                norm=f32(f"l{i}.norm1", (C,)), w_in=Dense(w_in, None, dev, md),
                w_out=Dense(w_out, out_b, dev, md), cols=cols, n_in=n, k_out=w_out.shape[1],
                conv_w=conv_w.contiguous().to(dev), conv_b=conv_b, A_log=A_log, dt_bias=dt_bias, mix_norm=mix_norm,
                skip=skip, gate_b=gate_b, up_b=up_b)
        m.embed = t("embed", (cfg.vocab, C)).to(md).contiguous().to(dev)
        m.final_norm = f32("final.norm", (C,))
        m.head = Dense(t("head", (cfg.vocab, C)), None, dev, md)
        return m

    # ------------------------------------------------------------------ forward
    def forward(self, fb, cache, ws: VugotarWorkspace) -> torch.Tensor:
        cfg = self.cfg
        T, C, eps = fb.T, cfg.hidden, cfg.rms_eps
        if T > ws.max_tokens:
            raise ValueError(f"step of {T} tokens, workspace holds {ws.max_tokens}")
        b16 = self.dtype != torch.float32
        rag = HY.Ragged(fb)
        x = ws.x[:T]
        HY.embed_rows(self.embed, fb.tokens, x)
        if fb.embed_rows:
            for r0, e in fb.embed_rows:
                x[r0:r0 + e.shape[0]].copy_(e)
        hin = ws.hin[:T]
        for ri, (li, add_embed) in enumerate(self.runs):
            if fb.stop_layer is not None and ri >= fb.stop_layer:
                break
            L, W = cfg.layers[li], self.weights[li]
            kv, state, tails = cache.layer(ri)
            if add_embed:
                HY.embed_rows(self.embed, fb.tokens, x, accumulate=True)
            HY.offset_rmsnorm(x, W.norm, eps, out32=None if b16 else hin, out16=hin if b16 else None)
            y = ws.y[:T * W.n_in].view(T, W.n_in)
            W.w_in.into(hin, y)
            cat = ws.cat[:T * W.k_out].view(T, W.k_out)
            c = W.cols
            if L.type == "parallel":
                k0 = self._left(L.mixer, y, c, fb, rag, kv, ws, cat, eps)
                k0 = self._right(L.mixer, W, y, c, rag, state, tails, ws, cat, k0, eps)
            else:
                k0 = self._mamba2(L.mixer, W, y, c, rag, state, tails, ws, cat, eps)
            f = L.mlp
            if f is not None and f.kind == "dense":
                HY.glu(y[:, c["gate"]:c["gate"] + f.ff], y[:, c["up"]:c["up"] + f.ff], W.gate_b, W.up_b,
                       cat[:, k0:k0 + f.ff])
            elif f is not None:
                if f.shared_ff:
                    Fs = f.shared_ff
                    HY.glu(y[:, c["sgate"]:c["sgate"] + Fs], y[:, c["sup"]:c["sup"] + Fs], None, None,
                           cat[:, k0:k0 + Fs], scale=y[:, c["sg"]:c["sg"] + 1], group=Fs, scale_sigmoid=True)
                    k0 += Fs
                E = f.experts
                rw = ws.route[:T * E].view(T, E)
                HY.moe_route(y[:, c["router"]:c["router"] + E], f.top, f.router_scale, rw, ROUTE_EPS)
                HY.glu(y[:, c["egate"]:c["egate"] + E * f.ff], y[:, c["eup"]:c["eup"] + E * f.ff], None, None,
                       cat[:, k0:k0 + E * f.ff], scale=rw, group=f.ff)
            W.w_out.acc(cat, x)
        if fb.stop_layer is not None:
            return x
        S = fb.logits_idx.numel()
        if S > ws.logits_rows:
            raise ValueError(f"{S} logit rows asked, workspace holds {ws.logits_rows}")
        hs = ws.hs[:S]
        HY.offset_rmsnorm(x, self.final_norm, eps, out32=None if b16 else hs, out16=hs if b16 else None,
                          rows=fb.logits_idx)
        if fb.want_hidden or fb.keep_hidden:
            if fb.want_hidden:
                return hs.float()
            self.last_hidden = hs.float()
        return self.head.into(hs, ws.logits[:S])

    def _left(self, mx: ParallelCfg, y, c, fb, rag, kv, ws, cat, eps) -> int:
        a = mx.left
        T = y.shape[0]
        H, G, dk, dv = a.heads, a.kv_heads, a.dim, a.vdim
        q = ws.q[:T * H * dk].view(T, H * dk)
        HY.rope_norm_append(y[:, c["lq"]:c["lq"] + H * dk], y[:, c["lk"]:c["lk"] + G * dk],
                            y[:, c["lv"]:c["lv"] + G * dv], fb.positions, H, G, dk, dv, a.rot_dims, a.rot_base, True,
                            eps, q, kv[0], kv[1], fb.slots)
        HY.masked_attention(q, kv[0], kv[1], rag, H, G, dk, dv, a.scale, cat[:, :H * dv], chunk=a.chunk, sink=True,
                            out_scale=mx.left_scale, workspace=(ws.part_ml, ws.part_o))
        return H * dv

    def _right(self, mx: ParallelCfg, W, y, c, rag, state, tails, ws, cat, k0: int, eps) -> int:
        r = mx.right
        T = y.shape[0]
        H, G, dk, dv = r.heads, r.kv_heads, r.dim, r.vdim
        nq, nv = G * dk, H * dv
        cc = 2 * nq + nv
        xc = ws.conv[:T * cc].view(T, cc)
        HY.causal_conv(y[:, c["rq"]:c["rq"] + cc], W.conv_w, None, tails, rag, xc, silu=True)
        HY.unit_norm_heads(xc[:, :2 * nq], 2 * G, dk, DELTA_UNIT_EPS, dk ** -0.5, split=G, scale2=1.0)  # q | k
        decay, coef = ws.decay[:T * H].view(T, H), ws.coef[:T * H].view(T, H)
        HY.scan_coefs(y[:, c["ra"]:c["ra"] + H], y[:, c["rb"]:c["rb"] + H], W.A_log, W.dt_bias, decay, coef)
        o = ws.scan[:T * nv].view(T, nv)
        HY.state_scan(xc[:, nq:2 * nq], xc[:, :nq], xc[:, 2 * nq:], decay, coef, None, state, rag, o, H, G, dk, dv,
                      delta=True)
        HY.gated_group_norm(o, y[:, c["rg"]:c["rg"] + nv], W.mix_norm, eps, dv, cat[:, k0:k0 + nv], gate_first=False,
                            out_scale=mx.right_scale)
        return k0 + nv

    def _mamba2(self, m: Mamba2Cfg, W, y, c, rag, state, tails, ws, cat, eps) -> int:
        T = y.shape[0]
        inner, gn, H = m.inner, m.groups * m.state, m.heads
        c0 = c["in"]
        cc = inner + 2 * gn
        xc = ws.conv[:T * cc].view(T, cc)
        HY.causal_conv(y[:, c0 + inner:c0 + inner + cc], W.conv_w, W.conv_b, tails, rag, xc, silu=True)
        decay, coef = ws.decay[:T * H].view(T, H), ws.coef[:T * H].view(T, H)
        HY.scan_coefs(y[:, c0 + inner + cc:c0 + inner + cc + H], None, W.A_log, W.dt_bias, decay, coef)
        o = ws.scan[:T * inner].view(T, inner)
        HY.state_scan(xc[:, inner:inner + gn], xc[:, inner + gn:], xc[:, :inner], decay, coef, W.skip, state, rag, o, H,
                      m.groups, m.state, m.vdim, delta=False)
        HY.gated_group_norm(o, y[:, c0:c0 + inner], W.mix_norm, eps, inner // m.norm_groups, cat[:, :inner],
                            gate_first=True)
        return inner


# ------------------------------------------------------------------------------------------------ sources
def is_vugotar_dir(path: str) -> bool:
    f = os.path.join(path, "config.json")
    if not (os.path.isdir(path) and os.path.isfile(f)):
        return False
    try:
        with open(f) as fh:
            return json.load(fh).get("architecture") == ARCH
    except (OSError, ValueError):
        return False


def dir_source(model_dir: str):
    """(VugotarConfig, get) of a directory holding config.json and model.safetensors."""
    from .vosotar import tensor_getter
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = VugotarConfig.from_json(json.load(f), os.path.basename(os.path.normpath(model_dir)))
    return cfg, tensor_getter(model_dir)


def tensor_shapes(cfg: VugotarConfig) -> dict:
    """name -> shape of every checkpoint tensor of a configuration."""
    C = cfg.hidden
    s = {"embed": (cfg.vocab, C), "final.norm": (C,), "head": (cfg.vocab, C)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", L.mixer
        s[f"l{i}.norm1"] = (C,)
        if L.type == "parallel":
            a, r = m.left, m.right
            s.update({p + "left.q": (a.heads * a.dim, C), p + "left.k": (a.kv_heads * a.dim, C),
                      p + "left.v": (a.kv_heads * a.vdim, C), p + "left.o": (C, a.heads * a.vdim),
                      p + "right.q": (r.kv_heads * r.dim, C), p + "right.q.conv": (r.kv_heads * r.dim, r.conv),
                      p + "right.k": (r.kv_heads * r.dim, C), p + "right.k.conv": (r.kv_heads * r.dim, r.conv),
                      p + "right.v": (r.heads * r.vdim, C), p + "right.v.conv": (r.heads * r.vdim, r.conv),
                      p + "right.b": (r.heads, C), p + "right.a": (r.heads, C), p + "right.A_log": (r.heads,),
                      p + "right.dt_bias": (r.heads,), p + "right.norm": (r.vdim,),
                      p + "right.g": (r.heads * r.vdim, C),
                      p + "right.o": (C, r.heads * r.vdim)})
        else:
            cc = m.inner + 2 * m.groups * m.state
            s.update({p + "in": (m.inner + cc + m.heads, C), p + "conv": (cc, m.conv), p + "conv.b": (cc,),
                      p + "dt_bias": (m.heads,), p + "A_log": (m.heads,), p + "D": (m.heads,), p + "norm": (m.inner,),
                      p + "o": (C, m.inner)})
        f, q = L.mlp, f"l{i}.mlp."
        if f is not None and f.kind == "dense":
            s.update({q + "gate": (f.ff, C), q + "gate.b": (f.ff,), q + "up": (f.ff, C), q + "up.b": (f.ff,),
                      q + "down": (C, f.ff), q + "down.b": (C,)})
        elif f is not None:
            for e in range(f.experts):
                s.update({f"{q}e{e}.gate": (f.ff, C), f"{q}e{e}.up": (f.ff, C), f"{q}e{e}.down": (C, f.ff)})
            s[q + "router"] = (f.experts, C)
            if f.shared_ff:
                s.update({q + "shared.gate": (f.shared_ff, C), q + "shared.up": (f.shared_ff, C),
                          q + "shared.down": (C, f.shared_ff), q + "shared.sg": (1, C)})
    return s


def synthetic_source(cfg: VugotarConfig, seed: int = 0):
    """Random weights (bf16-representable) under the checkpoint's tensor names, made on first use."""
    made: dict = {}
    sh = tensor_shapes(cfg)
    order = sorted(sh)

    def get(name):
        if name not in sh:
            return None
        if name not in made:
            g = torch.Generator().manual_seed(seed * 1000003 + order.index(name))
            s = sh[name]
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1",) or name == "final.norm":
                a = 0.1 * torch.randn(s, generator=g)
            elif leaf == "norm":
                a = 1.0 + 0.1 * torch.randn(s, generator=g)
            elif leaf == "A_log":
                a = torch.log(0.5 + 2.0 * torch.rand(s, generator=g))
            elif leaf == "dt_bias":
                a = torch.randn(s, generator=g) - 1.0
            elif leaf == "D":
                a = 1.0 + 0.2 * torch.randn(s, generator=g)
            elif leaf == "b":
                a = (0.5 if len(s) == 1 else s[-1] ** -0.5) * torch.randn(s, generator=g)
            elif leaf == "conv":
                a = 0.5 * torch.randn(s, generator=g)
            elif leaf == "router":
                a = 2.0 * torch.randn(s, generator=g) * (s[-1] ** -0.5)
            else:
                a = torch.randn(s, generator=g) * (s[-1] ** -0.5)
            made[name] = a.to(torch.bfloat16)
        return made[name]
    get.names = order
    return get


def save_checkpoint(cfg: VugotarConfig, get, model_dir: str) -> None:
    """Write config.json + model.safetensors (bf16) of `get`'s tensors: the layout `dir_source` reads."""
    from safetensors.torch import save_file
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: get(k).contiguous() for k in get.names}, os.path.join(model_dir, "model.safetensors"))


def load_dir(model_dir: str, device="cpu", dtype=None) -> VugotarModel:
    cfg, get = dir_source(model_dir)
    return VugotarModel.load(cfg, get, device, dtype)
