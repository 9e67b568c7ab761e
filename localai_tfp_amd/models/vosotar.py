"""Vosotar: a decoder whose layers mix tokens with latent attention (no positional rotation) and carry a short
causal convolution over each mixer's input.

One layer on the fp32 residual x (T rows of a ragged engine step; g* are one-number gains):

    h    = g1 * unit_rms(x)                              (latent.hip scalar norm -> fp32 + GEMM operand)
    gate = h W_rg1^T                                      (hipBLASLt, fp32 out; its bias joins in the gated add)
    hm   = h + tapconv(h)                                 (latent.hip; last taps-1 rows of h carried per sequence)
    y    = hm [W_dq | W_dkv | W_g]^T                      (one GEMM for the three projections that read hm)
    cq   = w_q * unit_rms(y[:, :q_rank]);  c = w_kv * unit_rms(y[:, q_rank:+rank]) -> paged latent pool
    qa   = (cq W_uq^T) per head times U_k                 (GEMM, then batched GEMM: absorbed queries [H, T, rank])
    o    = softmax(scale * qa . c_j) over j <= position, times c_j       (latent_attn.hip, keys = values = latents)
    att  = (o U_v^T) * sigmoid(y[:, gate columns]) per head              (batched GEMM, latent.hip pack)
    x   += g1b * unit_rms((att W_o^T) * sigmoid(gate + b)) (GEMM, latent.hip gated norm add)
    h2   = g2 * unit_rms(x);  u = h2 [W_up | W_rg2]^T
    x   += g2b * unit_rms((relu(u_up)^2 W_down^T) * sigmoid(u_rg2 + b2))

A layer entry may name another layer whose tensors it uses (`weights_of`); it still has its own latent pool and
convolution tails. A layer without a feed-forward stops after the mixer. Sizes come from config.json, per layer.

The engine sees `cache_kind = "latent"`: a paged pool of latents (block tables and flat slots as for K / V) plus one
state slot per live sequence for the convolution tails (engine/kv_cache.py LatentCache, SlotPool).

`dtype` bf16: GEMM operands and the cached latent are bf16, everything between GEMMs fp32. `dtype` fp32: all fp32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import torch

from ..ops import latent as LA
from ..ops.dense import Dense
from ..ops.dense import bmm_f32 as _bmm_f32

ARCH = "Vosotar"


@dataclass
class LatentMixer:
    heads: int
    dim: int  # query / key size per head
    vdim: int  # value size per head
    kv_rank: int
    q_rank: int
    scale: float


@dataclass
class VosotarLayerCfg:
    mixer: LatentMixer
    ff: int | None  # dense feed-forward width, None: no feed-forward
    weights_of: int | None = None
    type: str = "latent_attention"


@dataclass
class VosotarConfig:
    name: str = "vosotar"
    arch: str = "vosotar"
    hidden: int = 256
    vocab: int = 512
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    taps: int = 3
    ctx_train: int = 1 << 20  # no positions anywhere: the engine's max_model_len is the only limit
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

    @classmethod
    def from_json(cls, d: dict, name: str = "vosotar") -> "VosotarConfig":
        if d.get("architecture") != ARCH:
            raise ValueError(f"not a {ARCH} configuration")
        layers = []
        for i, e in enumerate(d["layers"]):
            if e["type"] != "latent_attention":
                raise ValueError(f"layer {i}: unknown mixer {e['type']!r}")
            m = e["mixer"]
            mlp = e.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward {mlp.get('kind')!r}")
            wo, hops = e.get("weights_of"), 0
            while wo is not None:  # follow a chain of borrowed layers to the one that has the tensors
                if not 0 <= int(wo) < len(d["layers"]) or hops > len(d["layers"]):
                    raise ValueError(f"layer {i}: weights_of does not lead to a layer with tensors of its own")
                nxt = d["layers"][int(wo)].get("weights_of")
                if nxt is None:
                    break
                wo, hops = nxt, hops + 1
            layers.append(VosotarLayerCfg(
                LatentMixer(int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), int(m["q_rank"]),
                            float(m["scale"])),
                int(mlp["ff"]) if mlp is not None else None, int(wo) if wo is not None else None))
        return cls(name=name, hidden=int(d["width"]), vocab=int(d["vocab"]), layers=layers,
                   rms_eps=float(d["norm"]["eps"]), taps=int(d["canon"]["taps"]))

    def to_json(self) -> dict:
        ls = []
        for L in self.layers:
            m = L.mixer
            e = {"type": L.type, "mixer": {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                                           "q_rank": m.q_rank, "scale": m.scale},
                 "mlp": {"kind": "dense", "ff": L.ff} if L.ff is not None else None}
            if L.weights_of is not None:
                e["weights_of"] = L.weights_of
            ls.append(e)
        return {"architecture": ARCH, "width": self.hidden, "vocab": self.vocab, "norm": {"eps": self.rms_eps},
                "canon": {"taps": self.taps}, "layers": ls}


def make_config(hidden=256, vocab=512, n_layers=2, heads=4, dim=32, vdim=32, kv_rank=64, q_rank=96, ff=512, taps=3,
                shared: int = 0, scale: float | None = None, eps: float = 1e-6, name="vosotar") -> VosotarConfig:
    """A uniform configuration: `n_layers` layers with tensors, then `shared` more that reuse them in order."""
    mk = lambda wo=None: VosotarLayerCfg(LatentMixer(heads, dim, vdim, kv_rank, q_rank,  # noqa: E731
                                                       float(scale if scale is not None else dim ** -0.5)), ff, wo)
    layers = [mk() for _ in range(n_layers)] + [mk(i % n_layers) for i in range(shared)]
    return VosotarConfig(name=name, hidden=hidden, vocab=vocab, layers=layers, rms_eps=eps, taps=taps)


# sizes of the order of a 1B / 7B decoder with a 512-wide latent (bench / synthetic checkpoints)
SYNTHETIC = {
    "vosotar-tiny": dict(hidden=256, vocab=512, n_layers=2, heads=4, dim=32, vdim=32, kv_rank=64, q_rank=96, ff=512),
    "vosotar-1b": dict(hidden=2048, vocab=32000, n_layers=16, heads=16, dim=128, vdim=128, kv_rank=512, q_rank=768,
                       ff=8192),
    "vosotar-7b": dict(hidden=4096, vocab=32000, n_layers=32, heads=32, dim=128, vdim=128, kv_rank=512, q_rank=1536,
                       ff=14336),
}


@dataclass
class VosotarWeights:
    """Device tensors of one layer that has tensors of its own."""
    n1: torch.Tensor
    n1b: torch.Tensor
    n2: torch.Tensor | None
    n2b: torch.Tensor | None
    canon: torch.Tensor  # [C, taps] fp32
    rg1: Dense  # [C, C]; its bias joins in the gated add
    rg1_b: torch.Tensor
    rg2_b: torch.Tensor | None
    w_in: Dense  # rows: dq | dkv | g
    dq_norm: torch.Tensor
    dkv_norm: torch.Tensor
    uq: Dense
    uk: torch.Tensor  # [H, dim, rank]
    uvt: torch.Tensor  # [H, rank, vdim]
    o: Dense
    up_rg2: Dense | None  # rows: up | rg2
    down: Dense | None


class VosotarWorkspace:
    """Step scratch sized for the largest step; forward() only takes views (static addresses for graph capture)."""

    def __init__(self, cfg: VosotarConfig, max_tokens: int, max_seqs: int, logits_rows: int, device, dtype,
                 max_parts: int = 64):
        dev = torch.device(device)
        T, C = max_tokens, cfg.hidden
        f32 = dict(dtype=torch.float32, device=dev)
        md = dict(dtype=dtype, device=dev)
        self.max_tokens, self.max_seqs = T, max_seqs
        self.logits_rows = S = max(max_seqs, logits_rows)
        ms = [L.mixer for L in cfg.layers]
        n_in = max(m.q_rank + m.kv_rank + m.heads for m in ms)
        ffc = max([L.ff + C for L in cfg.layers if L.ff is not None] or [C])
        ffm = max([L.ff for L in cfg.layers if L.ff is not None] or [1])
        self.h = torch.empty((T, C), **f32)
        self.h32 = torch.empty((T, C), **f32)
        self.h16 = torch.empty((T, C), **md)
        self.hm = torch.empty((T, C), **md)
        self.gate = torch.empty((T * C,), **f32)
        self.y = torch.empty((T * C,), **f32)
        self.y_in = torch.empty((T * n_in,), **f32)
        self.cq = torch.empty((T * max(m.q_rank for m in ms),), **md)
        self.q = torch.empty((T * max(m.heads * m.dim for m in ms),), **md)
        self.qa = torch.empty((T * max(m.heads * m.kv_rank for m in ms),), **md)
        self.ol = torch.empty((T * max(m.heads * m.kv_rank for m in ms),), **md)
        self.ov = torch.empty((T * max(m.heads * m.vdim for m in ms),), **f32)
        self.att = torch.empty((T * max(m.heads * m.vdim for m in ms),), **md)
        self.u = torch.empty((T * ffc,), **f32)
        self.act = torch.empty((T * ffm,), **md)
        self.hs = torch.empty((S, C), **md)
        self.logits = torch.empty((S, cfg.vocab), **f32)
        # partial results of decode rows whose keys are split into partitions: room for every sequence at
        # `max_parts` partitions, and for a lone sequence split finely enough to cover the chip
        hmax, rmax = max(m.heads for m in ms), max(m.kv_rank for m in ms)
        rows = hmax * max(max_seqs * max_parts, 256)
        self.part_ml = torch.empty((rows, 2), **f32)
        self.part_o = torch.empty((rows, rmax), **f32)


class VosotarModel:
    cache_kind = "latent"
    tp_size = 1
    n_kv = 1
    n_heads = 1
    DECODE_WGS = 512  # decode attention: workgroups to aim for when splitting contexts into key partitions

    def decode_part_len(self, n_dec: int, heads: int, max_len: int) -> int:
        """Keys per partition of the decode attention: a workgroup holds up to 64 (token, head) rows of one
        sequence, so few sequences with long contexts are split finely (down to one 32-key tile) to cover the CUs, and
        large batches coarsely (fewer partials to merge)."""
        wgs = max(1, n_dec * -(-heads // (32 if heads <= 32 else 64)))
        want = max(1, self.DECODE_WGS // wgs)  # partitions per sequence
        per = -(-max(1, max_len) // want)
        return max(32, -(-per // 32) * 32)

    def __init__(self, cfg: VosotarConfig, device="cpu", dtype=None):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype is None:
            dtype = torch.bfloat16 if self.device.type == "cuda" else torch.float32
        if self.device.type != "cuda":
            dtype = torch.float32  # the CPU plumbing path runs everything in fp32
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Vosotar runs in bfloat16 or float32")
        self.dtype = dtype
        self.weights: dict[int, VosotarWeights] = {}
        self.embed: torch.Tensor | None = None
        self.embed_norm = self.final_norm = None
        self.head: Dense | None = None
        self.last_hidden = None

    # ------------------------------------------------------------------ engine hooks
    def make_cache(self, num_blocks: int, block_size: int, state_slots: int):
        from ..engine.kv_cache import LatentCache
        c = self.cfg
        return LatentCache([L.mixer.kv_rank for L in c.layers], num_blocks, block_size, self.device, self.dtype,
                           state_slots, c.taps - 1, c.hidden)

    def cache_ranks(self):
        return [L.mixer.kv_rank for L in self.cfg.layers]

    def make_workspace(self, max_tokens: int, max_seqs: int, logits_rows: int = 0, max_parts: int = 64):
        return VosotarWorkspace(self.cfg, max_tokens, max_seqs, logits_rows, self.device, self.dtype, max_parts)

    def weight_bytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size() + self.head.w.numel() * self.head.w.element_size()
        for W in self.weights.values():
            for d in (W.rg1, W.w_in, W.uq, W.o, W.up_rg2, W.down):
                if d is not None:
                    n += d.w.numel() * d.w.element_size()
            n += (W.uk.numel() + W.uvt.numel()) * W.uk.element_size()
        return n

    # ------------------------------------------------------------------ loading
    @classmethod
    def load(cls, cfg: VosotarConfig, get, device="cpu", dtype=None) -> "VosotarModel":
        """`get(name)` -> torch tensor (any float dtype) of the checkpoint tensor `name`."""
        m = cls(cfg, device, dtype)
        dev, md = m.device, m.dtype
        C = cfg.hidden

        def t(name, shape=None):
            a = get(name)
            if a is None:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            if shape is not None and tuple(a.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(a.shape)}, configuration says {tuple(shape)}")
            return a

        def f32(name, shape=None):
            return t(name, shape).to(torch.float32).reshape(-1 if shape in (None, ()) else shape).contiguous().to(dev)

        def one(name):
            return t(name).to(torch.float32).reshape(1).contiguous().to(dev)

        for i, L in enumerate(cfg.layers):
            if L.weights_of is not None:
                continue
            p, mx = f"l{i}.", L.mixer
            H, d, dv, R, Rq = mx.heads, mx.dim, mx.vdim, mx.kv_rank, mx.q_rank
            w_in = torch.cat([t(p + "mix.dq", (Rq, C)).float(), t(p + "mix.dkv", (R, C)).float(),
                              t(p + "mix.g", (H, C)).float()], 0)
            uk = t(p + "mix.uk", (H * d, R)).float().reshape(H, d, R)
            uv = t(p + "mix.uv", (H * dv, R)).float().reshape(H, dv, R)
            up_rg2 = down = n2 = n2b = rg2_b = None
            if L.ff is not None:
                up_rg2 = Dense(torch.cat([t(p + "mlp.up", (L.ff, C)).float(), t(p + "rg2", (C, C)).float()], 0),
                               None, dev, md)
                rg2_b = f32(p + "rg2.b", (C,))
                down = Dense(t(p + "mlp.down", (C, L.ff)).float(), None, dev, md)
                n2, n2b = one(p + "norm2"), one(p + "norm2b")
            m.weights[i] = VosotarWeights(
                n1=one(p + "norm1"), n1b=one(p + "norm1b"), n2=n2, n2b=n2b,
                canon=f32(p + "canon1", (C, cfg.taps)),
                rg1=Dense(t(p + "rg1", (C, C)).float(), None, dev, md), rg1_b=f32(p + "rg1.b", (C,)), rg2_b=rg2_b,
                w_in=Dense(w_in, None, dev, md),
                dq_norm=f32(p + "mix.dq.norm", (Rq,)), dkv_norm=f32(p + "mix.dkv.norm", (R,)),
                uq=Dense(t(p + "mix.uq", (H * d, Rq)).float(), None, dev, md),
                uk=uk.to(dev).to(md).contiguous(), uvt=uv.transpose(1, 2).to(dev).to(md).contiguous(),
                o=Dense(t(p + "mix.o", (C, H * dv)).float(), None, dev, md),
                up_rg2=up_rg2, down=down)
        for i, L in enumerate(cfg.layers):  # a layer that borrows tensors must agree with their sizes
            if L.weights_of is not None and (L.mixer != cfg.layers[L.weights_of].mixer or
                                             L.ff != cfg.layers[L.weights_of].ff):
                raise ValueError(f"layer {i}: sizes differ from layer {L.weights_of}, whose tensors it uses")
        m.embed = t("embed", (cfg.vocab, C)).to(md).contiguous().to(dev)
        m.embed_norm, m.final_norm = one("embed.norm"), one("final.norm")
        m.head = Dense(t("head", (cfg.vocab, C)).float(), None, dev, md)
        return m

    # ------------------------------------------------------------------ forward
    def forward(self, fb, cache, ws: VosotarWorkspace) -> torch.Tensor:
        cfg = self.cfg
        T, C, eps = fb.T, cfg.hidden, cfg.rms_eps
        if T > ws.max_tokens:
            raise ValueError(f"step of {T} tokens, workspace holds {ws.max_tokens}")
        b16 = self.dtype != torch.float32
        rag = LA.Ragged(fb)
        x = ws.h[:T]
        LA.embed_scalar_norm(self.embed, fb.tokens, self.embed_norm, eps, x)
        if fb.embed_rows:
            for r0, e in fb.embed_rows:
                x[r0:r0 + e.shape[0]].copy_(e)
        h32 = ws.h32[:T]
        hin = ws.h16[:T] if b16 else h32
        hm = ws.hm[:T]
        gate = ws.gate[:T * C].view(T, C)
        y = ws.y[:T * C].view(T, C)
        normed = False  # h32 / hin already hold this layer's first norm
        for li, L in enumerate(cfg.layers):
            if fb.stop_layer is not None and li >= fb.stop_layer:
                break
            W = self.weights[L.weights_of if L.weights_of is not None else li]
            mx = L.mixer
            H, d, dv, R, Rq = mx.heads, mx.dim, mx.vdim, mx.kv_rank, mx.q_rank
            lat, tails = cache.layer(li)
            # ---- mixer ----
            if not normed:  # (otherwise the previous layer's last gated add wrote this norm in its own pass)
                LA.scalar_rmsnorm(x, W.n1, eps, out32=h32, out16=hin if b16 else None)
            W.rg1.into(hin, gate)
            LA.tap_conv(h32, W.canon, tails, rag, hm)
            n_in = Rq + R + H
            y_in = ws.y_in[:T * n_in].view(T, n_in)
            W.w_in.into(hm, y_in)
            cq = ws.cq[:T * Rq].view(T, Rq)
            LA.latent_norm_append(y_in, Rq, R, W.dq_norm, W.dkv_norm, eps, cq, lat, fb.slots)
            q = ws.q[:T * H * d].view(T, H * d)
            torch.mm(cq, W.uq.wt, out=q)
            qa = ws.qa[:H * T * R].view(H, T, R)
            torch.bmm(q.view(T, H, d).transpose(0, 1), W.uk, out=qa)
            ol = ws.ol[:H * T * R].view(H, T, R)
            LA.latent_attention(qa, lat, rag, mx.scale, ol, workspace=(ws.part_ml, ws.part_o),
                                part_len=self.decode_part_len(rag.n_dec, H, rag.dec_max_len) if rag.n_dec else 0)
            ov = ws.ov[:H * T * dv].view(H, T, dv)
            _bmm_f32(ol, W.uvt, ov)
            att = ws.att[:T * H * dv].view(T, H * dv)
            LA.head_gate_pack(ov, y_in[:, Rq + R:], att)
            W.o.into(att, y)
            # the norm that follows a gated add (this layer's feed-forward norm, or the next layer's first norm) is
            # written by the add's own pass
            nxt = cfg.layers[li + 1] if li + 1 < len(cfg.layers) and (fb.stop_layer is None or li + 1 < fb.stop_layer) \
                else None
            Wn = self.weights[nxt.weights_of if nxt.weights_of is not None else li + 1] if nxt is not None else None
            if L.ff is None:
                LA.gated_norm_add(x, y, gate, W.n1b, eps, W.rg1_b, next_g=Wn.n1 if Wn is not None else None,
                                  next32=h32, next16=hin if b16 else None)
                normed = Wn is not None
                continue
            LA.gated_norm_add(x, y, gate, W.n1b, eps, W.rg1_b, next_g=W.n2, next32=None if b16 else h32,
                              next16=hin if b16 else None)
            # ---- feed-forward ----
            F_ = L.ff
            u = ws.u[:T * (F_ + C)].view(T, F_ + C)
            W.up_rg2.into(hin, u)
            act = ws.act[:T * F_].view(T, F_)
            LA.relu2(u[:, :F_], act)
            W.down.into(act, y)
            LA.gated_norm_add(x, y, u[:, F_:], W.n2b, eps, W.rg2_b, next_g=Wn.n1 if Wn is not None else None,
                              next32=h32, next16=hin if b16 else None)
            normed = Wn is not None
        if fb.stop_layer is not None:
            return x
        # ---- head ----
        S = fb.logits_idx.numel()
        if S > ws.logits_rows:
            raise ValueError(f"{S} logit rows asked, workspace holds {ws.logits_rows}")
        hs = ws.hs[:S]
        LA.scalar_rmsnorm(x, self.final_norm, eps, out32=None if b16 else hs, out16=hs if b16 else None,
                          rows=fb.logits_idx)
        if fb.want_hidden or fb.keep_hidden:
            if fb.want_hidden:
                return hs.float()
            self.last_hidden = hs.float()
        return self.head.into(hs, ws.logits[:S])


# ------------------------------------------------------------------------------------------------ sources
def is_vosotar_dir(path: str) -> bool:
    f = os.path.join(path, "config.json")
    if not (os.path.isdir(path) and os.path.isfile(f)):
        return False
    try:
        with open(f) as fh:
            return json.load(fh).get("architecture") == ARCH
    except (OSError, ValueError):
        return False


def tensor_getter(model_dir: str):
    """get(name) -> tensor or None over every *.safetensors file of a directory (opened lazily, read by name)."""
    from safetensors import safe_open
    files = [os.path.join(model_dir, fn) for fn in sorted(os.listdir(model_dir)) if fn.endswith(".safetensors")]
    handles = [safe_open(fn, framework="pt") for fn in files]
    where = {k: h for h in handles for k in h.keys()}

    def get(name):
        h = where.get(name)
        return h.get_tensor(name) if h is not None else None
    return get


def dir_source(model_dir: str):
    """(VosotarConfig, get) of a directory holding config.json and model.safetensors."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = VosotarConfig.from_json(json.load(f), os.path.basename(os.path.normpath(model_dir)))
    return cfg, tensor_getter(model_dir)


def synthetic_source(cfg: VosotarConfig, seed: int = 0):
    """Random weights (bf16-representable) under the checkpoint's tensor names, made on first use."""
    made: dict = {}
    C = cfg.hidden

    def shapes():
        s = {"embed": (cfg.vocab, C), "embed.norm": (), "final.norm": (), "head": (cfg.vocab, C)}
        for i, L in enumerate(cfg.layers):
            if L.weights_of is not None:
                continue
            p, m = f"l{i}.", L.mixer
            s.update({p + "norm1": (), p + "norm1b": (), p + "canon1": (C, cfg.taps), p + "rg1": (C, C),
                      p + "rg1.b": (C,), p + "mix.dq": (m.q_rank, C), p + "mix.dq.norm": (m.q_rank,),
                      p + "mix.uq": (m.heads * m.dim, m.q_rank), p + "mix.dkv": (m.kv_rank, C),
                      p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                      p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads, C),
                      p + "mix.o": (C, m.heads * m.vdim)})
            if L.ff is not None:
                s.update({p + "norm2": (), p + "norm2b": (), p + "mlp.up": (L.ff, C), p + "mlp.down": (C, L.ff),
                          p + "rg2": (C, C), p + "rg2.b": (C,)})
        return s
    sh = shapes()

    def get(name):
        if name not in sh:
            return None
        if name not in made:
            g = torch.Generator().manual_seed(seed * 1000003 + sorted(sh).index(name))
            s = sh[name]
            if s == () or name.endswith(".norm"):
                a = 1.0 + 0.1 * torch.randn(s, generator=g)
            elif name.endswith(".b"):
                a = 0.5 * torch.randn(s, generator=g)
            elif name.endswith("canon1"):
                a = 0.3 * torch.randn(s, generator=g)
            else:
                a = torch.randn(s, generator=g) * (s[-1] ** -0.5)
            made[name] = a.to(torch.bfloat16)
        return made[name]
    get.names = sorted(sh)
    return get


def save_checkpoint(cfg: VosotarConfig, get, model_dir: str) -> None:
    """Write config.json + model.safetensors (bf16) of `get`'s tensors: the layout `dir_source` reads."""
    from safetensors.torch import save_file
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: get(k).contiguous() for k in get.names}, os.path.join(model_dir, "model.safetensors"))


def load_dir(model_dir: str, device="cpu", dtype=None) -> VosotarModel:
    cfg, get = dir_source(model_dir)
    return VosotarModel.load(cfg, get, device, dtype)
