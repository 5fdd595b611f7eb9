"""Keronex: a pre-norm decoder whose residual is kept as several streams (hyper-connections) and whose layers draw
their mixer from three kinds.

Embedding: x = scale * embed[token] + bigram[(prev * mul_prev + token * mul_cur) mod buckets]; a sequence's first token
has no token before it and takes the table's extra last row. The token before a step's first row is carried per
sequence (engine/kv_cache.py HybridCache.last_token).

Residual: S streams x_1 .. x_S, all equal to the embedding at the start. For sublayer f with weights in [S], out [S],
mix [S, S] (indexed [from, to]) and norm weight w:

    u   = sum_s in[s] x_s;      y = f(u / sqrt(mean(u^2) + eps) * (1 + w))
    x_t <- sum_s mix[s, t] x_s + out[t] y          all t at once, from the old streams

and the model's output reads the sum of the streams. Without `streams` in the configuration the same code runs one
stream with in = out = mix = 1: the plain pre-norm residual.

Mixers (`type`):
  attention      differential attention: every query head and key head carries two maps of `dim` numbers; each map is a
                 causal softmax attention of its own over the SAME values (grouped key / value heads), and a head's
                 output is unit_rms(a1 - lam * a2) * (1 - diff) with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one
                 number per layer. Rotary positions on the pairs (i, i + rot.dims / 2) of each map.
  retention      linear attention with a fixed decay per head and no softmax: S <- decay_h S + k v^T, o = S^T q with
                 rotary positions on q and k, k scaled by dim^-1/2; o is unit-RMS-normed per head, times silu(W_g h).
  channel_delta  gated delta rule with a decay per head and key channel: q, k, v pass a short causal convolution and a
                 SiLU, q and k become unit vectors; S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
                 with g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 h) + dt_bias)), beta = sigmoid(W_b h); o is
                 unit-RMS-normed per head, times a weight and sigmoid(W_g2 (W_g1 h)).
Feed-forward: `dense` = W_down (gelu_tanh(W_gate h) * (W_up h)); `moe` = sigmoid router scores, the `top` largest keep
their scores as weights (not renormalised) and multiply the expert's INPUT; experts and the always-on shared expert are
W_down relu(W_up h)^2. A layer with `weights_of: j` runs layer j's tensors on a cache and state of its own.

How a sublayer maps onto launches (T rows of a ragged engine step):

    hyper_step            the previous sublayer's stream update + this one's weighted sum + norm -> hin      1 launch
    y = hin W_in^T        every projection of the sublayer stacked into ONE GEMM (fp32 out)
    attention:     rotary + paged append (both maps' keys, one set of values); masked attention with twice the heads
                   (map-major, so the grouped-head rule holds per map) reading value head g % G; a1 - lam a2 + norm
    retention:     rotary in place on q | k; state scan with a constant decay per head; head norm * silu(g)
    channel_delta: convolution (q | k | v) + tails; unit norms; per-channel decays (second projection in fp32 inside);
                   state scan (delta rule, per-channel decay, sigmoid of the write strength while staging);
                   head norm * weight * sigmoid(second gate projection, fp32 inside)
    dense:         gelu_tanh GLU        moe: routing weights [T, E]; relu(w z)^2 for the shared and for every expert
    o = cat W_out^T       one GEMM; experts stacked along K, so the sum over experts is the GEMM's accumulator

An expert's input scaling commutes with its first projection (W_up (w h) = w (W_up h)), so all experts' first
projections stay one GEMM over the unscaled h and the weight enters before the squared ReLU.

The engine sees `cache_kind = "hybrid"`: paged key / value pools for the attention layers, one state slot per live
sequence for recurrent states, convolution tails and the previous token. `dtype` bf16: GEMM operands and the pools are
bf16, everything between GEMMs fp32. `dtype` fp32: all fp32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import torch

from ..ops import hybrid as HY
from ..ops.dense import Dense

ARCH = "Keronex"
UNIT_EPS = 1e-6  # inside the root of the delta rule's unit vectors


@dataclass
class DiffAttnCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    rot_dims: int = 0
    rot_base: float = 10000.0


@dataclass
class RetentionCfg:
    heads: int
    dim: int
    vdim: int
    decay: list
    rot_dims: int = 0
    rot_base: float = 10000.0


@dataclass
class ChannelDeltaCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    rank_a: int  # inner sizes of the decay's and the gate's two projections (the tensors' shapes give them)
    rank_g: int


@dataclass
class FfCfg:
    kind: str  # dense | moe
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: int | None = None


@dataclass
class KeronexLayerCfg:
    type: str  # attention | retention | channel_delta
    mixer: DiffAttnCfg | RetentionCfg | ChannelDeltaCfg
    mlp: FfCfg | None
    weights_of: int | None = None


def _need(cond: bool, what: str):
    if not cond:
        raise ValueError(f"Keronex configuration: {what}")


@dataclass
class KeronexConfig:
    name: str = "keronex"
    arch: str = "keronex"
    hidden: int = 256
    vocab: int = 512
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    emb_scale: float = 1.0
    bigram: tuple | None = None  # (buckets, mul_prev, mul_cur)
    streams: int | None = None  # None: one plain residual, no hyper-connection tensors
    ctx_train: int = 1 << 20
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

    def owner(self, i: int) -> int:
        """Index of the layer whose tensors layer i runs."""
        j = self.layers[i].weights_of
        return i if j is None else j

    @classmethod
    def from_json(cls, d: dict, name: str = "keronex", shapes=None) -> "KeronexConfig":
        """`shapes(tensor name)` -> shape gives the sizes config.json leaves to the tensors (inner sizes of the low-rank
        decay and gate projections); without it they come from the optional keys `rank_a` and `rank_g`."""
        if d.get("architecture") != ARCH:
            raise ValueError(f"not a {ARCH} configuration")

        def size(key, m, tensor, i):
            if key in m:
                return int(m[key])
            _need(shapes is not None, f"layer {i}: {key} is given by the shape of {tensor}")
            return int(shapes(tensor)[0])

        def rot(m):
            r = m.get("rot") or {}
            return int(r.get("dims", 0)), float(r.get("base", 10000.0))

        layers = []
        for i, e in enumerate(d["layers"]):
            m, src = e["mixer"], e.get("weights_of")
            j = i if src is None else int(src)
            if src is not None:
                _need(0 <= j < i and layers[j].weights_of is None,
                      f"layer {i}: weights_of names an earlier layer with tensors")
                _need(e["type"] == layers[j].type, f"layer {i}: same mixer as layer {j}")
            if e["type"] == "attention":
                mixer = DiffAttnCfg(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                    float(m["diff"]), *rot(m))
                _need(mixer.heads % mixer.kv_heads == 0, f"layer {i}: heads are a multiple of kv_heads")
            elif e["type"] == "retention":
                mixer = RetentionCfg(int(m["heads"]), int(m["dim"]), int(m["vdim"]), [float(x) for x in m["decay"]],
                                     *rot(m))
                _need(len(mixer.decay) == mixer.heads, f"layer {i}: one decay per head")
            elif e["type"] == "channel_delta":
                kvh = int(m.get("kv_heads", m["heads"]))
                mixer = ChannelDeltaCfg(int(m["heads"]), kvh, int(m["dim"]), int(m["vdim"]), int(m["conv"]),
                                        size("rank_a", m, f"l{j}.mix.a1", i), size("rank_g", m, f"l{j}.mix.g1", i))
                _need(mixer.heads % mixer.kv_heads == 0, f"layer {i}: heads are a multiple of kv_heads")
                _need(mixer.conv >= 1, f"layer {i}: at least one tap")
            else:
                raise ValueError(f"layer {i}: unknown mixer {e['type']!r}")
            if e["type"] != "channel_delta":
                _need(mixer.rot_dims % 2 == 0 and mixer.rot_dims <= mixer.dim, f"layer {i}: rot.dims even, at most dim")
            f = e.get("mlp")
            if f is None:
                mlp = None
            elif f.get("kind") == "dense":
                mlp = FfCfg("dense", int(f["ff"]))
            elif f.get("kind") == "moe":
                r, sh = f["router"], f.get("shared")
                mlp = FfCfg("moe", int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(sh["ff"]) if sh else None)
                _need(0 < mlp.top <= mlp.experts, f"layer {i}: 1 <= top <= experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward {f.get('kind')!r}")
            if src is not None:
                _need(mixer == layers[j].mixer and mlp == layers[j].mlp, f"layer {i}: the entry equals layer {j}'s")
            layers.append(KeronexLayerCfg(e["type"], mixer, mlp, None if src is None else j))
        emb = d.get("embedding") or {}
        bg = emb.get("bigram")
        streams = d.get("streams")
        if streams is not None:
            _need(1 <= int(streams) <= HY.HYPER_MAX_STREAMS, f"1 to {HY.HYPER_MAX_STREAMS} streams")
        return cls(name=name, hidden=int(d["width"]), vocab=int(d["vocab"]), layers=layers,
                   rms_eps=float(d["norm"]["eps"]), emb_scale=float(emb.get("scale", 1.0)),
                   bigram=(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None,
                   streams=None if streams is None else int(streams))

    def to_json(self) -> dict:
        ls = []
        for L in self.layers:
            m = L.mixer
            if L.type == "attention":
                mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                      "diff": m.diff}
            elif L.type == "retention":
                mj = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay)}
            else:
                mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            if L.type != "channel_delta" and m.rot_dims:
                mj["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
            f, fj = L.mlp, None
            if f is not None and f.kind == "dense":
                fj = {"kind": "dense", "ff": f.ff}
            elif f is not None:
                fj = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
                if f.shared_ff:
                    fj["shared"] = {"ff": f.shared_ff}
            e = {"type": L.type, "mixer": mj, "mlp": fj}
            if L.weights_of is not None:
                e["weights_of"] = L.weights_of
            ls.append(e)
        emb = {"scale": self.emb_scale}
        if self.bigram:
            emb["bigram"] = {"buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]}
        d = {"architecture": ARCH, "width": self.hidden, "vocab": self.vocab, "norm": {"eps": self.rms_eps},
             "embedding": emb, "layers": ls}
        if self.streams is not None:
            d["streams"] = self.streams
        return d


def make_config(hidden=128, vocab=320, pattern=("retention", "attention", "channel_delta"), heads=4, kv_heads=2, dim=32,
                vdim=32, scale=None, diff=0.25, rot_dims=None, rot_base=10000.0, r_heads=4, r_dim=32, r_vdim=32,
                decay=None, r_rot_dims=None, d_heads=4, d_kv_heads=4, d_dim=32, d_vdim=32, conv=4, rank_a=8, rank_g=8,
                mlps=("dense", "moe"), ff=512, experts=4, top=2, expert_ff=128, shared_ff=128, weights_of=None,
                streams=3, emb_scale=1.0, bigram=(61, 7, 3), eps=1e-6, name="keronex") -> KeronexConfig:
    """A configuration whose i-th layer has mixer pattern[i] and feed-forward mlps[i % len(mlps)] ("dense" | "moe" |
    None); `weights_of` maps a layer index to the earlier layer whose tensors it runs."""
    layers = []
    for i, t in enumerate(pattern):
        j = (weights_of or {}).get(i)
        if j is not None:
            layers.append(KeronexLayerCfg(layers[j].type, layers[j].mixer, layers[j].mlp, j))
            continue
        if t == "attention":
            mixer = DiffAttnCfg(heads, kv_heads, dim, vdim, float(scale if scale is not None else dim ** -0.5),
                                float(diff), dim if rot_dims is None else rot_dims, float(rot_base))
        elif t == "retention":
            dl = list(decay) if decay is not None else [1.0 - 2.0 ** (-5.0 - 4.0 * h / max(1, r_heads - 1))
                                                         for h in range(r_heads)]
            mixer = RetentionCfg(r_heads, r_dim, r_vdim, dl, r_dim if r_rot_dims is None else r_rot_dims, float(rot_base))
        else:
            mixer = ChannelDeltaCfg(d_heads, d_kv_heads, d_dim, d_vdim, conv, rank_a, rank_g)
        k = mlps[i % len(mlps)]
        mlp = None if k is None else FfCfg("dense", ff) if k == "dense" else \
            FfCfg("moe", expert_ff, experts, top, shared_ff or None)
        layers.append(KeronexLayerCfg(t, mixer, mlp))
    return KeronexConfig(name=name, hidden=hidden, vocab=vocab, layers=layers, rms_eps=eps, emb_scale=float(emb_scale),
                         bigram=tuple(bigram) if bigram else None, streams=streams)


# sizes of the order of a 1B / 7B decoder (bench / synthetic checkpoints): two delta-rule layers, an attention layer
# and a retention layer in turn, on four streams
_PAT = ("channel_delta", "channel_delta", "attention", "retention")
SYNTHETIC = {
    "keronex-tiny": dict(hidden=192, vocab=384, pattern=("retention", "attention", "channel_delta", "retention"),
                         weights_of={3: 0}, streams=2),
    "keronex-1b": dict(hidden=2048, vocab=32000, pattern=_PAT * 4, heads=16, kv_heads=4, dim=64, vdim=128, r_heads=16,
                       r_dim=128, r_vdim=128, d_heads=16, d_kv_heads=16, d_dim=128, d_vdim=128, rank_a=32, rank_g=32,
                       mlps=("dense", "moe", "moe", "moe"), ff=8192, experts=8, top=2, expert_ff=2048, shared_ff=4096,
                       streams=4, bigram=(65521, 1009, 31)),
    "keronex-7b": dict(hidden=4096, vocab=32000, pattern=_PAT * 8, heads=32, kv_heads=8, dim=64, vdim=128, r_heads=32,
                       r_dim=128, r_vdim=128, d_heads=32, d_kv_heads=32, d_dim=128, d_vdim=128, rank_a=32, rank_g=32,
                       mlps=("dense", "moe", "moe", "moe"), ff=14336, experts=8, top=2, expert_ff=3584, shared_ff=7168,
                       streams=4, bigram=(65521, 1009, 31)),
}


@dataclass
class KeronexWeights:
    """Device tensors of one layer, with the column layout of its stacked GEMMs."""
    norm1: torch.Tensor
    hc1: tuple  # (in [S], out [S], mix [S, S]) fp32
    w_in: Dense
    w_o: Dense
    cols: dict  # name -> first column of the projection in the input GEMM's output
    n_in: int
    k_o: int
    lam: float = 0.0  # attention: exp(lq1 . lk1) - exp(lq2 . lk2) + diff
    decay: torch.Tensor | None = None  # retention: one constant per head
    conv_w: torch.Tensor | None = None
    a2: torch.Tensor | None = None  # [rank_a, heads * dim], fp32 in both modes
    dt_bias: torch.Tensor | None = None
    A_log: torch.Tensor | None = None
    g2: torch.Tensor | None = None  # [rank_g, heads * vdim], fp32 in both modes
    mix_norm: torch.Tensor | None = None
    norm2: torch.Tensor | None = None
    hc2: tuple | None = None
    w_ff: Dense | None = None
    w_down: Dense | None = None
    ff_cols: dict | None = None
    n_ff: int = 0
    k_down: int = 0


class KeronexWorkspace:
    """Step scratch sized for the largest step; forward() only takes views (static addresses for graph capture)."""

    def __init__(self, model: "KeronexModel", max_tokens: int, max_seqs: int, logits_rows: int):
        cfg, dev, md = model.cfg, model.device, model.dtype
        T, C, S = max_tokens, cfg.hidden, cfg.streams or 1
        f32 = dict(dtype=torch.float32, device=dev)
        m16 = dict(dtype=md, device=dev)
        self.max_tokens, self.max_seqs = T, max_seqs
        self.logits_rows = R = max(max_seqs, logits_rows)
        Ws = list(model.weights.values())
        n_y = max(max(W.n_in, W.n_ff) for W in Ws)
        k_cat = max(max(W.k_o, W.k_down) for W in Ws)
        n_q = n_att = n_conv = n_dec = n_scan = n_e = 1
        for L in cfg.layers:
            m = L.mixer
            if L.type == "attention":
                n_q = max(n_q, 2 * m.heads * m.dim)
                n_att = max(n_att, 2 * m.heads * m.vdim)
            elif L.type == "retention":
                n_scan = max(n_scan, m.heads * m.vdim)
            else:
                n_conv = max(n_conv, 2 * m.kv_heads * m.dim + m.heads * m.vdim)
                n_dec = max(n_dec, m.heads * m.dim)
                n_scan = max(n_scan, m.heads * m.vdim)
            if L.mlp is not None and L.mlp.kind == "moe":
                n_e = max(n_e, L.mlp.experts)
        self.xs = torch.empty((T, S * C), **f32)
        self.x = torch.empty((T, C), **f32)
        self.hin = torch.empty((T, C), **m16)
        self.y = torch.empty((T * n_y,), **f32)
        self.o = torch.empty((T, C), **f32)
        self.q = torch.empty((T * n_q,), **m16)
        self.att = torch.empty((T * n_att,), **f32)
        self.conv = torch.empty((T * n_conv,), **f32)
        self.decay = torch.empty((T * n_dec,), **f32)
        self.scan = torch.empty((T * n_scan,), **f32)
        self.cat = torch.zeros((T * k_cat,), **m16)  # zero: padded columns are read, never written
        self.route = torch.empty((T * n_e,), **f32)
        self.hs = torch.empty((R, C), **m16)
        self.logits = torch.empty((R, cfg.vocab), **f32)
        att = [L.mixer for L in cfg.layers if L.type == "attention"]
        rows = HY.DECODE_WAVES + max_seqs * max([2 * a.heads for a in att] or [1])
        self.part_ml = torch.empty((rows, 2), **f32)
        self.part_o = torch.empty((rows, max([a.vdim for a in att] or [1])), **f32)


class KeronexModel:
    cache_kind = "hybrid"
    tp_size = 1
    n_kv = 1
    n_heads = 1

    def __init__(self, cfg: KeronexConfig, device="cpu", dtype=None):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype is None:
            dtype = torch.bfloat16 if self.device.type == "cuda" else torch.float32
        if self.device.type != "cuda":
            dtype = torch.float32  # the CPU plumbing path runs everything in fp32
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Keronex runs in bfloat16 or float32")
        self.dtype = dtype
        self.weights: dict[int, KeronexWeights] = {}
        self.embed: torch.Tensor | None = None
        self.pair: torch.Tensor | None = None
        self.final_norm = None
        self.head: Dense | None = None
        self.last_hidden = None

    # ------------------------------------------------------------------ engine hooks
    def cache_spec(self) -> list:
        spec = []
        for L in self.cfg.layers:
            m = L.mixer
            if L.type == "attention":  # both maps' keys, one set of values
                spec.append({"kv": (2 * m.kv_heads * m.dim, m.kv_heads * m.vdim)})
            elif L.type == "retention":
                spec.append({"state": (m.heads, m.vdim, m.dim)})
            else:
                spec.append({"state": (m.heads, m.vdim, m.dim),
                             "tails": (m.conv - 1, 2 * m.kv_heads * m.dim + m.heads * m.vdim)})
        return spec

    def make_cache(self, num_blocks: int, block_size: int, state_slots: int):
        from ..engine.kv_cache import HybridCache
        return HybridCache(self.cache_spec(), num_blocks, block_size, self.device, self.dtype, state_slots,
                           seq_tokens=self.cfg.bigram is not None)

    def cache_ranks(self):
        """Pool numbers per token of every attention layer."""
        return [sum(e["kv"]) for e in self.cache_spec() if e.get("kv")]

    def make_workspace(self, max_tokens: int, max_seqs: int, logits_rows: int = 0, max_parts: int = 64):
        return KeronexWorkspace(self, max_tokens, max_seqs, logits_rows)

    def weight_bytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size() + self.head.w.numel() * self.head.w.element_size()
        if self.pair is not None:
            n += self.pair.numel() * self.pair.element_size()
        for W in self.weights.values():
            for dn in (W.w_in, W.w_o, W.w_ff, W.w_down):
                if dn is not None:
                    n += dn.w.numel() * dn.w.element_size()
            for t in (W.a2, W.g2, W.conv_w):
                if t is not None:
                    n += t.numel() * 4
        return n

    # ------------------------------------------------------------------ loading
    @classmethod
    def load(cls, cfg: KeronexConfig, get, device="cpu", dtype=None) -> "KeronexModel":
        """`get(name)` -> torch tensor (any float dtype) of the checkpoint tensor `name`."""
        m = cls(cfg, device, dtype)
        dev, md = m.device, m.dtype
        C, S = cfg.hidden, cfg.streams

        def t(name, shape):
            a = get(name)
            if a is None:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            if tuple(a.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(a.shape)}, configuration says {tuple(shape)}")
            return a.float()

        def f32(name, shape):
            return t(name, shape).contiguous().to(dev)

        def stack(parts):
            """[(key, weight)] -> (weight rows padded to whole 16-byte rows, first column of each key, row count)."""
            cols, n = {}, 0
            for key, w in parts:
                cols[key] = n
                n += w.shape[0]
            w = torch.cat([w for _, w in parts], 0)
            if n % 8:
                w = torch.cat([w, torch.zeros(8 - n % 8, C)], 0)
            return w, cols, w.shape[0]

        def along_k(outs):
            w = torch.cat(outs, 1)
            if w.shape[1] % 8:  # the padded columns of the operand are never written and stay zero
                w = torch.cat([w, torch.zeros(C, 8 - w.shape[1] % 8)], 1)
            return w

        def hyper(prefix):
            if S is None:  # one plain residual: x <- x + y, read as it is
                one = torch.ones(1, dtype=torch.float32, device=dev)
                return one, one, one.view(1, 1)
            return f32(prefix + ".in", (S,)), f32(prefix + ".out", (S,)), f32(prefix + ".mix", (S, S))

        def maps_first(w, n, dk):
            """Rows [head][map][dk] -> [map][head][dk]: per map the heads lie as an ordinary grouped-head layout."""
            return w.view(n, 2, dk, C).transpose(0, 1).reshape(2 * n * dk, C)

        for i, L in enumerate(cfg.layers):
            if L.weights_of is not None:
                continue
            p, mx = f"l{i}.mix.", L.mixer
            kw = {}
            if L.type == "attention":
                H, G, dk, dv = mx.heads, mx.kv_heads, mx.dim, mx.vdim
                parts = [("q", maps_first(t(p + "q", (2 * H * dk, C)), H, dk)),
                         ("k", maps_first(t(p + "k", (2 * G * dk, C)), G, dk)), ("v", t(p + "v", (G * dv, C)))]
                lq1, lk1, lq2, lk2 = (t(p + n, (dk,)) for n in ("lq1", "lk1", "lq2", "lk2"))
                kw["lam"] = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + mx.diff)
                w_o = along_k([t(p + "o", (C, H * dv))])
            elif L.type == "retention":
                H, dk, dv = mx.heads, mx.dim, mx.vdim
                parts = [("q", t(p + "q", (H * dk, C))), ("k", t(p + "k", (H * dk, C))), ("v", t(p + "v", (H * dv, C))),
                         ("g", t(p + "g", (H * dv, C)))]
                kw["decay"] = torch.tensor(mx.decay, dtype=torch.float32, device=dev)
                w_o = along_k([t(p + "o", (C, H * dv))])
            else:
                H, G, dk, dv, ra, rg = mx.heads, mx.kv_heads, mx.dim, mx.vdim, mx.rank_a, mx.rank_g
                parts = [("q", t(p + "q", (G * dk, C))), ("k", t(p + "k", (G * dk, C))), ("v", t(p + "v", (H * dv, C))),
                         ("b", t(p + "b", (H, C))), ("a1", t(p + "a1", (ra, C))), ("g1", t(p + "g1", (rg, C)))]
                conv_w = torch.cat([t(p + "q.conv", (G * dk, mx.conv)), t(p + "k.conv", (G * dk, mx.conv)),
                                    t(p + "v.conv", (H * dv, mx.conv))], 0)
                kw.update(conv_w=conv_w.contiguous().to(dev), a2=t(p + "a2", (H * dk, ra)).t().contiguous().to(dev),
                          dt_bias=f32(p + "dt_bias", (H * dk,)), A_log=f32(p + "A_log", (H,)),
                          g2=t(p + "g2", (H * dv, rg)).t().contiguous().to(dev), mix_norm=f32(p + "norm", (dv,)))
                w_o = along_k([t(p + "o", (C, H * dv))])
            w_in, cols, n_in = stack(parts)
            f, q = L.mlp, f"l{i}.mlp."
            if f is not None:
                if f.kind == "dense":
                    fparts = [("gate", t(q + "gate", (f.ff, C))), ("up", t(q + "up", (f.ff, C)))]
                    outs = [t(q + "down", (C, f.ff))]
                else:
                    fparts, outs = [("router", t(q + "router", (f.experts, C)))], []
                    if f.shared_ff:
                        fparts.append(("sup", t(q + "shared.up", (f.shared_ff, C))))
                        outs.append(t(q + "shared.down", (C, f.shared_ff)))
                    fparts.append(("eup", torch.cat([t(f"{q}e{e}.up", (f.ff, C)) for e in range(f.experts)], 0)))
                    outs += [t(f"{q}e{e}.down", (C, f.ff)) for e in range(f.experts)]
                w_ff, ff_cols, n_ff = stack(fparts)
                w_down = along_k(outs)
                kw.update(norm2=f32(f"l{i}.norm2", (C,)), hc2=hyper(f"l{i}.hc2"), w_ff=Dense(w_ff, None, dev, md),
                          w_down=Dense(w_down, None, dev, md), ff_cols=ff_cols, n_ff=n_ff, k_down=w_down.shape[1])
            m.weights[i] = KeronexWeights(norm1=f32(f"l{i}.norm1", (C,)), hc1=hyper(f"l{i}.hc1"),
                                          w_in=Dense(w_in, None, dev, md), w_o=Dense(w_o, None, dev, md), cols=cols,
                                          n_in=n_in, k_o=w_o.shape[1], **kw)
        m.embed = t("embed", (cfg.vocab, C)).to(md).contiguous().to(dev)
        if cfg.bigram:
            m.pair = t("bigram", (cfg.bigram[0] + 1, C)).to(md).contiguous().to(dev)
        m.final_norm = f32("final.norm", (C,))
        m.head = Dense(t("head", (cfg.vocab, C)), None, dev, md)
        return m

    # ------------------------------------------------------------------ forward
    def forward(self, fb, cache, ws: KeronexWorkspace) -> torch.Tensor:
        cfg = self.cfg
        T, C, eps, S = fb.T, cfg.hidden, cfg.rms_eps, cfg.streams or 1
        if T > ws.max_tokens:
            raise ValueError(f"step of {T} tokens, workspace holds {ws.max_tokens}")
        if fb.embed_rows:
            raise NotImplementedError("Keronex takes token ids only")
        b16 = self.dtype != torch.float32
        rag = HY.Ragged(fb)
        xs, hin, o = ws.xs[:T], ws.hin[:T], ws.o[:T]
        h32, h16 = (None, hin) if b16 else (hin, None)
        bg = cfg.bigram or (1, 0, 0)
        HY.embed_pair(self.embed, self.pair, fb.tokens, rag, cache.last_token, cfg.emb_scale, bg[1], bg[2], bg[0], xs,
                      copies=S)
        pend = (None, None, None)  # (output, mix, out weights) of the sublayer whose stream update is still to do
        for li, L in enumerate(cfg.layers):
            if fb.stop_layer is not None and li >= fb.stop_layer:
                break
            W = self.weights[cfg.owner(li)]
            kv, state, tails = cache.layer(li)
            HY.hyper_step(xs, pend[0], pend[1], pend[2], W.hc1[0], W.norm1, eps, h32, h16)
            y = ws.y[:T * W.n_in].view(T, W.n_in)
            W.w_in.into(hin, y)
            cat = ws.cat[:T * W.k_o].view(T, W.k_o)
            if L.type == "attention":
                self._attention(L.mixer, W, y, fb, rag, kv, ws, cat, eps)
            elif L.type == "retention":
                self._retention(L.mixer, W, y, fb, rag, state, ws, cat, eps)
            else:
                self._channel_delta(L.mixer, W, y, rag, state, tails, ws, cat, eps)
            W.w_o.into(cat, o)
            pend = (o, W.hc1[2], W.hc1[1])
            f = L.mlp
            if f is None:
                continue
            HY.hyper_step(xs, o, W.hc1[2], W.hc1[1], W.hc2[0], W.norm2, eps, h32, h16)
            c = W.ff_cols
            y = ws.y[:T * W.n_ff].view(T, W.n_ff)
            W.w_ff.into(hin, y)
            cat = ws.cat[:T * W.k_down].view(T, W.k_down)
            if f.kind == "dense":
                HY.glu(y[:, c["gate"]:c["gate"] + f.ff], y[:, c["up"]:c["up"] + f.ff], None, None, cat[:, :f.ff],
                       act="gelu_tanh")
            else:
                k0 = 0
                if f.shared_ff:
                    k0 = f.shared_ff
                    HY.glu(y[:, c["sup"]:c["sup"] + k0], None, None, None, cat[:, :k0], act="relu2")
                E = f.experts
                rw = ws.route[:T * E].view(T, E)
                HY.moe_route(y[:, c["router"]:c["router"] + E], f.top, 1.0, rw, 0.0, mode="sigmoid")
                HY.glu(y[:, c["eup"]:c["eup"] + E * f.ff], None, None, None, cat[:, k0:k0 + E * f.ff], scale=rw,
                       group=f.ff, act="relu2")
            W.w_down.into(cat, o)
            pend = (o, W.hc2[2], W.hc2[1])
        x = ws.x[:T]
        HY.hyper_step(xs, pend[0], pend[1], pend[2], None, None, eps, total=x)
        if fb.stop_layer is not None:
            return x
        R = fb.logits_idx.numel()
        if R > ws.logits_rows:
            raise ValueError(f"{R} logit rows asked, workspace holds {ws.logits_rows}")
        hs = ws.hs[:R]
        HY.offset_rmsnorm(x, self.final_norm, eps, out32=None if b16 else hs, out16=hs if b16 else None,
                          rows=fb.logits_idx)
        if fb.want_hidden or fb.keep_hidden:
            if fb.want_hidden:
                return hs.float()
            self.last_hidden = hs.float()
        return self.head.into(hs, ws.logits[:R])

    def _attention(self, a: DiffAttnCfg, W, y, fb, rag, kv, ws, cat, eps):
        T = y.shape[0]
        H, G, dk, dv = a.heads, a.kv_heads, a.dim, a.vdim
        c = W.cols
        q = ws.q[:T * 2 * H * dk].view(T, 2 * H * dk)
        # twice the heads, map-major: query head m H + h reads key head m G + h // (H / G) and value head h // (H / G)
        HY.rope_norm_append(y[:, c["q"]:c["q"] + 2 * H * dk], y[:, c["k"]:c["k"] + 2 * G * dk],
                            y[:, c["v"]:c["v"] + G * dv], fb.positions, 2 * H, 2 * G, dk, dv, a.rot_dims, a.rot_base,
                            False, eps, q, kv[0], kv[1], fb.slots, half=True, v_heads=G)
        att = ws.att[:T * 2 * H * dv].view(T, 2 * H * dv)
        HY.masked_attention(q, kv[0], kv[1], rag, 2 * H, 2 * G, dk, dv, a.scale, att,
                            workspace=(ws.part_ml, ws.part_o), v_heads=G, p32=True)
        HY.diff_group_norm(att[:, :H * dv], att[:, H * dv:], W.lam, eps, dv, cat[:, :H * dv], out_scale=1.0 - a.diff)

    def _retention(self, r: RetentionCfg, W, y, fb, rag, state, ws, cat, eps):
        T = y.shape[0]
        H, dk, dv = r.heads, r.dim, r.vdim
        c = W.cols
        nk, nv = H * dk, H * dv
        HY.rope_rows(y[:, c["q"]:c["q"] + 2 * nk], fb.positions, 2 * H, dk, r.rot_dims, r.rot_base, half=True,
                     scale=1.0, split=H, scale2=dk ** -0.5)  # q | k lie side by side
        o = ws.scan[:T * nv].view(T, nv)
        HY.state_scan(y[:, c["k"]:c["k"] + nk], y[:, c["q"]:c["q"] + nk], y[:, c["v"]:c["v"] + nv], W.decay, None, None,
                      state, rag, o, H, H, dk, dv, delta=False)
        HY.gated_group_norm(o, y[:, c["g"]:c["g"] + nv], None, eps, dv, cat[:, :nv], gate_first=False)

    def _channel_delta(self, d: ChannelDeltaCfg, W, y, rag, state, tails, ws, cat, eps):
        T = y.shape[0]
        H, G, dk, dv = d.heads, d.kv_heads, d.dim, d.vdim
        c = W.cols
        nq, nv = G * dk, H * dv
        cc = 2 * nq + nv
        xc = ws.conv[:T * cc].view(T, cc)
        HY.causal_conv(y[:, c["q"]:c["q"] + cc], W.conv_w, None, tails, rag, xc, silu=True)
        HY.unit_norm_heads(xc[:, :2 * nq], 2 * G, dk, UNIT_EPS, dk ** -0.5, split=G, scale2=1.0)  # q | k
        decay = ws.decay[:T * H * dk].view(T, H * dk)
        HY.channel_decay(y[:, c["a1"]:c["a1"] + d.rank_a], W.dt_bias, 1.0, decay, proj=W.a2, rate_log=W.A_log)
        o = ws.scan[:T * nv].view(T, nv)
        HY.state_scan(xc[:, nq:2 * nq], xc[:, :nq], xc[:, 2 * nq:], decay, y[:, c["b"]:c["b"] + H], None, state, rag, o,
                      H, G, dk, dv, delta=True, channel=True, coef_sigmoid=True)
        HY.gated_group_norm(o, y[:, c["g1"]:c["g1"] + d.rank_g], W.mix_norm, eps, dv, cat[:, :nv], gate_first=False,
                            act="sigmoid", proj=W.g2)


# ------------------------------------------------------------------------------------------------ sources
def is_keronex_dir(path: str) -> bool:
    f = os.path.join(path, "config.json")
    if not (os.path.isdir(path) and os.path.isfile(f)):
        return False
    try:
        with open(f) as fh:
            return json.load(fh).get("architecture") == ARCH
    except (OSError, ValueError):
        return False


def dir_source(model_dir: str):
    """(KeronexConfig, get) of a directory holding config.json and model.safetensors."""
    from .vosotar import tensor_getter
    get = tensor_getter(model_dir)

    def shapes(name):
        a = get(name)
        if a is None:
            raise KeyError(f"checkpoint has no tensor {name!r}")
        return tuple(a.shape)
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = KeronexConfig.from_json(json.load(f), os.path.basename(os.path.normpath(model_dir)), shapes)
    return cfg, get


def tensor_shapes(cfg: KeronexConfig) -> dict:
    """name -> shape of every checkpoint tensor of a configuration."""
    C, S = cfg.hidden, cfg.streams
    s = {"embed": (cfg.vocab, C), "final.norm": (C,), "head": (cfg.vocab, C)}
    if cfg.bigram:
        s["bigram"] = (cfg.bigram[0] + 1, C)
    for i, L in enumerate(cfg.layers):
        if L.weights_of is not None:
            continue
        p, m = f"l{i}.mix.", L.mixer
        subs = ["1"]
        s[f"l{i}.norm1"] = (C,)
        if L.type == "attention":
            s.update({p + "q": (2 * m.heads * m.dim, C), p + "k": (2 * m.kv_heads * m.dim, C),
                      p + "v": (m.kv_heads * m.vdim, C), p + "o": (C, m.heads * m.vdim)})
            s.update({p + n: (m.dim,) for n in ("lq1", "lk1", "lq2", "lk2")})
        elif L.type == "retention":
            s.update({p + "q": (m.heads * m.dim, C), p + "k": (m.heads * m.dim, C), p + "v": (m.heads * m.vdim, C),
                      p + "g": (m.heads * m.vdim, C), p + "o": (C, m.heads * m.vdim)})
        else:
            nq, nv = m.kv_heads * m.dim, m.heads * m.vdim
            s.update({p + "q": (nq, C), p + "q.conv": (nq, m.conv), p + "k": (nq, C), p + "k.conv": (nq, m.conv),
                      p + "v": (nv, C), p + "v.conv": (nv, m.conv), p + "b": (m.heads, C), p + "A_log": (m.heads,),
                      p + "norm": (m.vdim,), p + "a1": (m.rank_a, C), p + "a2": (m.heads * m.dim, m.rank_a),
                      p + "dt_bias": (m.heads * m.dim,), p + "g1": (m.rank_g, C), p + "g2": (nv, m.rank_g),
                      p + "o": (C, nv)})
        f, q = L.mlp, f"l{i}.mlp."
        if f is not None:
            subs.append("2")
            s[f"l{i}.norm2"] = (C,)
            if f.kind == "dense":
                s.update({q + "gate": (f.ff, C), q + "up": (f.ff, C), q + "down": (C, f.ff)})
            else:
                for e in range(f.experts):
                    s.update({f"{q}e{e}.up": (f.ff, C), f"{q}e{e}.down": (C, f.ff)})
                s[q + "router"] = (f.experts, C)
                if f.shared_ff:
                    s.update({q + "shared.up": (f.shared_ff, C), q + "shared.down": (C, f.shared_ff)})
        if S is not None:
            for n in subs:
                s.update({f"l{i}.hc{n}.in": (S,), f"l{i}.hc{n}.out": (S,), f"l{i}.hc{n}.mix": (S, S)})
    return s


def synthetic_source(cfg: KeronexConfig, seed: int = 0):
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
            if ".hc" in name:
                n = s[0]
                if leaf == "in":
                    a = 1.0 / n + 0.1 * torch.randn(s, generator=g)
                elif leaf == "out":
                    a = 1.0 + 0.2 * torch.randn(s, generator=g)
                else:  # near the identity, so the streams neither die nor blow up over the layers
                    a = 0.8 * torch.eye(n) + 0.2 / n + 0.05 * torch.randn(s, generator=g)
            elif leaf in ("norm1", "norm2") or name == "final.norm":
                a = 0.1 * torch.randn(s, generator=g)
            elif leaf == "norm":
                a = 1.0 + 0.1 * torch.randn(s, generator=g)
            elif leaf in ("lq1", "lk1", "lq2", "lk2"):
                a = 0.3 * torch.randn(s, generator=g)
            elif leaf == "A_log":
                a = torch.log(0.5 + 2.0 * torch.rand(s, generator=g))
            elif leaf == "dt_bias":
                a = torch.randn(s, generator=g) - 3.0  # decays near one, as a trained layer keeps them
            elif leaf == "conv":
                a = 0.5 * torch.randn(s, generator=g)
            elif leaf == "router":
                a = 2.0 * torch.randn(s, generator=g) * (s[-1] ** -0.5)
            elif name in ("embed", "bigram"):
                a = torch.randn(s, generator=g)
            else:
                a = torch.randn(s, generator=g) * (s[-1] ** -0.5)
            made[name] = a.to(torch.bfloat16)
        return made[name]
    get.names = order
    return get


def save_checkpoint(cfg: KeronexConfig, get, model_dir: str) -> None:
    """Write config.json + model.safetensors (bf16) of `get`'s tensors: the layout `dir_source` reads."""
    from safetensors.torch import save_file
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: get(k).contiguous() for k in get.names}, os.path.join(model_dir, "model.safetensors"))


def load_dir(model_dir: str, device="cpu", dtype=None) -> KeronexModel:
    cfg, get = dir_source(model_dir)
    return KeronexModel.load(cfg, get, device, dtype)
