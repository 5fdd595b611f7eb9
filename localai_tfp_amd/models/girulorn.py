"""Girulorn: a decoder whose sublayers read the fp32 residual itself and whose norms sit on the sublayers' OUTPUTS:

    x += rms_norm_1(mixer(x))
    x += rms_norm_2(ff(x))                  (absent when the layer has no feed-forward)

Mixers (`type`):
  attention  softmax attention with grouped key/value heads and NO rotation. Queries and keys pass an RMS norm per
             head (one weight vector shared by the heads); the query at position p is multiplied by the temperature
             1 + coef * ln(floor((p + 1) / every) + 1); score = scale * q.k + rel[bucket(i - j), h], a learned bias per
             distance bucket and head (exact buckets for near keys, logarithmic ones up to `bias_max`); the softmax
             denominator holds one more term exp(sink_h) that carries no value; head h's output is multiplied by
             sigmoid((W_g x)_h) before the output projection. A layer with `kv_from: j` has no key / value tensors:
             it attends over layer j's paged keys and values with its own queries, bias, sinks and gate.
  gla        gated linear attention: per head S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t with q scaled by
             dim^-1/2 and a decay per key channel alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau); o is RMS-normed per head,
             multiplied by silu(W_g x) and projected. The state is fp32 [dim, vdim] per head and sequence.
Feed-forward (`mlp.kind` = moe): router logits W_r x + b in fp32, the `top` largest chosen, weights = softmax over the
chosen logits alone; experts and the shared expert are W_down (silu(W_gate x) * (W_up x)) without biases.
Logits = head (rms_norm_final(x)).

How a layer maps onto launches (T rows of a ragged engine step; hin is x in fp32 mode, its bf16 rounding otherwise):

    y = hin W_in^T              every projection of the mixer that reads x, stacked into ONE GEMM (fp32 out)
    attention: head norms + temperature + paged append; masked attention (bias, sink, gate fused) -> cat
    gla:       channel decays (second decay projection in fp32 + bias + sigmoid^(1/tau)); state scan; head norm * silu(g)
               -> cat
    o = cat W_o^T (fp32);  x += norm(o), hin <- x                                 ops/hybrid.py norm_add
    y = hin W_ff^T              router | shared gate, up | every expert's gate, up as ONE GEMM
    routing weights [T, E]; glu (shared); glu (experts, each scaled by its routing weight, 0 when not chosen) -> cat
    o = cat W_down^T            shared down and every expert's down stacked along K, so the weighted sum over
                                experts and the shared expert's addition happen in the GEMM's accumulator
    x += norm(o), hin <- x

The engine sees `cache_kind = "hybrid"`: paged key / value pools for every attention layer that owns keys, plus one
state slot per live sequence for the recurrent states (engine/kv_cache.py HybridCache, SlotPool).
`dtype` bf16: GEMM operands and the pools are bf16, everything between GEMMs fp32 (the decay's second projection
stays fp32: its input is the fp32 accumulator of the first). `dtype` fp32: all fp32.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import torch

from ..ops import hybrid as HY
from ..ops.dense import Dense

ARCH = "Girulorn"


@dataclass
class BiasAttnCfg:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float
    bias_rows: int  # rows of the distance-bias table (a tensor's shape gives it)
    temp_coef: float = 0.0
    temp_every: int = 1
    kv_from: int | None = None


@dataclass
class GlaCfg:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int  # inner size of the decay's two projections


@dataclass
class MoeCfg:
    ff: int
    experts: int
    top: int
    shared_ff: int | None = None


@dataclass
class GirulornLayerCfg:
    type: str  # attention | gla
    mixer: BiasAttnCfg | GlaCfg
    mlp: MoeCfg | None


def _need(cond: bool, what: str):
    if not cond:
        raise ValueError(f"Girulorn configuration: {what}")


@dataclass
class GirulornConfig:
    name: str = "girulorn"
    arch: str = "girulorn"
    hidden: int = 256
    vocab: int = 512
    layers: list = field(default_factory=list)
    rms_eps: float = 1e-6
    ctx_train: int = 1 << 20  # no positional table: the engine's max_model_len is the limit
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
    def from_json(cls, d: dict, name: str = "girulorn", shapes=None) -> "GirulornConfig":
        """`shapes(tensor name)` -> shape gives the sizes config.json leaves to the tensors (rows of the distance-bias
        table, inner size of the decay projections); without it they come from the optional keys `bias_rows` and
        `rank`."""
        if d.get("architecture") != ARCH:
            raise ValueError(f"not a {ARCH} configuration")

        def size(key, m, tensor, axis, i):
            if key in m:
                return int(m[key])
            _need(shapes is not None, f"layer {i}: {key} is given by the shape of {tensor}")
            return int(shapes(tensor)[axis])

        layers = []
        for i, e in enumerate(d["layers"]):
            m = e["mixer"]
            if e["type"] == "attention":
                qt = m.get("q_temp") or {}
                src = m.get("kv_from")
                mixer = BiasAttnCfg(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                    float(m["bias_max"]), size("bias_rows", m, f"l{i}.mix.rel", 0, i),
                                    float(qt.get("coef", 0.0)), int(qt.get("every", 1)),
                                    None if src is None else int(src))
                _need(mixer.heads % mixer.kv_heads == 0, f"layer {i}: heads are a multiple of kv_heads")
                _need(mixer.temp_every >= 1, f"layer {i}: q_temp.every >= 1")
                _need(mixer.bias_rows >= 2 and mixer.bias_max > mixer.bias_rows // 2,
                      f"layer {i}: at least two bias rows, bias_max beyond the exact half")
                if mixer.kv_from is not None:
                    j = mixer.kv_from
                    _need(0 <= j < i and layers[j].type == "attention" and layers[j].mixer.kv_from is None,
                          f"layer {i}: kv_from names an earlier attention layer with keys of its own")
                    o = layers[j].mixer
                    _need((o.kv_heads, o.dim, o.vdim) == (mixer.kv_heads, mixer.dim, mixer.vdim),
                          f"layer {i}: key / value sizes equal those of layer {j}")
            elif e["type"] == "gla":
                mixer = GlaCfg(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]),
                               size("rank", m, f"l{i}.mix.a1", 0, i))
                _need(mixer.tau > 0, f"layer {i}: tau > 0")
            else:
                raise ValueError(f"layer {i}: unknown mixer {e['type']!r}")
            f = e.get("mlp")
            if f is None:
                mlp = None
            elif f.get("kind") == "moe":
                r, sh = f["router"], f.get("shared")
                mlp = MoeCfg(int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(sh["ff"]) if sh else None)
                _need(0 < mlp.top <= mlp.experts, f"layer {i}: 1 <= top <= experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward {f.get('kind')!r}")
            layers.append(GirulornLayerCfg(e["type"], mixer, mlp))
        return cls(name=name, hidden=int(d["width"]), vocab=int(d["vocab"]), layers=layers,
                   rms_eps=float(d["norm"]["eps"]))

    def to_json(self) -> dict:
        ls = []
        for L in self.layers:
            m = L.mixer
            if L.type == "attention":
                mj = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                      "bias_max": m.bias_max, "q_temp": {"coef": m.temp_coef, "every": m.temp_every}}
                if m.kv_from is not None:
                    mj["kv_from"] = m.kv_from
            else:
                mj = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau}
            f = L.mlp
            fj = None
            if f is not None:
                fj = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
                if f.shared_ff:
                    fj["shared"] = {"ff": f.shared_ff}
            ls.append({"type": L.type, "mixer": mj, "mlp": fj})
        return {"architecture": ARCH, "width": self.hidden, "vocab": self.vocab, "norm": {"eps": self.rms_eps},
                "layers": ls}


def make_config(hidden=256, vocab=512, pattern=("attention", "gla"), heads=4, kv_heads=2, dim=32, vdim=32, scale=None,
                bias_max=100.0, bias_rows=16, temp_coef=0.25, temp_every=32, kv_from=None, g_heads=4, g_dim=32,
                g_vdim=32, tau=8.0, rank=8, mlps=("moe",), experts=4, top=2, expert_ff=128, shared_ff=128, eps=1e-6,
                name="girulorn") -> GirulornConfig:
    """A configuration whose i-th layer has mixer pattern[i] and feed-forward mlps[i % len(mlps)] ("moe" | None);
    `kv_from` maps a layer index to the attention layer whose keys and values it reads."""
    layers = []
    for i, t in enumerate(pattern):
        if t == "attention":
            mixer = BiasAttnCfg(heads, kv_heads, dim, vdim, float(scale if scale is not None else dim ** -0.5),
                                float(bias_max), bias_rows, temp_coef, temp_every, (kv_from or {}).get(i))
        else:
            mixer = GlaCfg(g_heads, g_dim, g_vdim, float(tau), rank)
        k = mlps[i % len(mlps)]
        layers.append(GirulornLayerCfg(t, mixer, None if k is None else MoeCfg(expert_ff, experts, top, shared_ff or None)))
    return GirulornConfig(name=name, hidden=hidden, vocab=vocab, layers=layers, rms_eps=eps)


# sizes of the order of a 1B / 7B decoder (bench / synthetic checkpoints): attention and gated-linear-attention layers
# in turn, every second attention layer reading the keys and values of the one before it
SYNTHETIC = {
    "girulorn-tiny": dict(hidden=256, vocab=512, pattern=("attention", "gla", "attention"), kv_from={2: 0}),
    "girulorn-1b": dict(hidden=2048, vocab=32000, pattern=("attention", "gla") * 8, heads=16, kv_heads=4, dim=128,
                        vdim=128, bias_max=4096.0, bias_rows=64, temp_every=1024, g_heads=16, g_dim=128, g_vdim=128,
                        tau=12.0, rank=32, experts=8, top=2, expert_ff=2048, shared_ff=4096,
                        kv_from={i: i - 2 for i in range(2, 16, 4)}),
    "girulorn-7b": dict(hidden=4096, vocab=32000, pattern=("attention", "gla") * 16, heads=32, kv_heads=8, dim=128,
                        vdim=128, bias_max=4096.0, bias_rows=64, temp_every=1024, g_heads=32, g_dim=128, g_vdim=128,
                        tau=12.0, rank=32, experts=8, top=2, expert_ff=3584, shared_ff=7168,
                        kv_from={i: i - 2 for i in range(2, 32, 4)}),
}


@dataclass
class GirulornWeights:
    """Device tensors of one layer, with the column layout of its stacked GEMMs."""
    norm1: torch.Tensor
    w_in: Dense
    w_o: Dense
    cols: dict  # name -> first column of the projection in the input GEMM's output
    n_in: int
    k_o: int
    q_norm: torch.Tensor | None = None
    k_norm: torch.Tensor | None = None
    bias: torch.Tensor | None = None  # distance-bias table, one entry per head and distance [H, ceil(bias_max) + 1]
    sink: torch.Tensor | None = None
    a2: torch.Tensor | None = None  # [rank, heads * dim], fp32 in both modes
    a2_b: torch.Tensor | None = None
    mix_norm: torch.Tensor | None = None
    norm2: torch.Tensor | None = None
    w_ff: Dense | None = None
    w_down: Dense | None = None
    ff_cols: dict | None = None
    n_ff: int = 0
    k_down: int = 0
    router_b: torch.Tensor | None = None


class GirulornWorkspace:
    """Step scratch sized for the largest step; forward() only takes views (static addresses for graph capture)."""

    def __init__(self, model: "GirulornModel", max_tokens: int, max_seqs: int, logits_rows: int):
        cfg, dev, md = model.cfg, model.device, model.dtype
        T, C = max_tokens, cfg.hidden
        f32 = dict(dtype=torch.float32, device=dev)
        m16 = dict(dtype=md, device=dev)
        self.max_tokens, self.max_seqs = T, max_seqs
        self.logits_rows = S = max(max_seqs, logits_rows)
        Ws = list(model.weights.values())
        n_y = max(max(W.n_in, W.n_ff) for W in Ws)
        k_cat = max(max(W.k_o, W.k_down) for W in Ws)
        n_q = n_dec = n_scan = n_e = 1
        for L in cfg.layers:
            m = L.mixer
            if L.type == "attention":
                n_q = max(n_q, m.heads * m.dim)
            else:
                n_dec = max(n_dec, m.heads * m.dim)
                n_scan = max(n_scan, m.heads * m.vdim)
            if L.mlp is not None:
                n_e = max(n_e, L.mlp.experts)
        self.x = torch.empty((T, C), **f32)
        self.hin = torch.empty((T, C), **m16) if md != torch.float32 else None  # fp32 mode: the GEMMs read x itself
        self.y = torch.empty((T * n_y,), **f32)
        self.o = torch.empty((T, C), **f32)
        self.q = torch.empty((T * n_q,), **m16)
        self.decay = torch.empty((T * n_dec,), **f32)
        self.scan = torch.empty((T * n_scan,), **f32)
        self.cat = torch.zeros((T * k_cat,), **m16)  # zero: padded columns are read, never written
        self.route = torch.empty((T * n_e,), **f32)
        self.hs = torch.empty((S, C), **m16)
        self.logits = torch.empty((S, cfg.vocab), **f32)
        att = [L.mixer for L in cfg.layers if L.type == "attention"]
        rows = HY.DECODE_WAVES + max_seqs * max([a.heads for a in att] or [1])
        self.part_ml = torch.empty((rows, 2), **f32)
        self.part_o = torch.empty((rows, max([a.vdim for a in att] or [1])), **f32)


class GirulornModel:
    cache_kind = "hybrid"
    tp_size = 1
    n_kv = 1
    n_heads = 1

    def __init__(self, cfg: GirulornConfig, device="cpu", dtype=None):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype is None:
            dtype = torch.bfloat16 if self.device.type == "cuda" else torch.float32
        if self.device.type != "cuda":
            dtype = torch.float32  # the CPU plumbing path runs everything in fp32
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Girulorn runs in bfloat16 or float32")
        self.dtype = dtype
        self.weights: dict[int, GirulornWeights] = {}
        self.embed: torch.Tensor | None = None
        self.final_norm = None
        self.head: Dense | None = None
        self.last_hidden = None

    # ------------------------------------------------------------------ engine hooks
    def cache_spec(self) -> list:
        spec = []
        for L in self.cfg.layers:
            m = L.mixer
            if L.type == "attention":
                spec.append({} if m.kv_from is not None else {"kv": (m.kv_heads * m.dim, m.kv_heads * m.vdim)})
            else:
                spec.append({"state": (m.heads, m.vdim, m.dim)})
        return spec

    def make_cache(self, num_blocks: int, block_size: int, state_slots: int):
        from ..engine.kv_cache import HybridCache
        return HybridCache(self.cache_spec(), num_blocks, block_size, self.device, self.dtype, state_slots)

    def cache_ranks(self):
        """Pool numbers per token of every layer that owns keys and values."""
        return [sum(e["kv"]) for e in self.cache_spec() if e.get("kv")]

    def make_workspace(self, max_tokens: int, max_seqs: int, logits_rows: int = 0, max_parts: int = 64):
        return GirulornWorkspace(self, max_tokens, max_seqs, logits_rows)

    def weight_bytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size() + self.head.w.numel() * self.head.w.element_size()
        for W in self.weights.values():
            for dn in (W.w_in, W.w_o, W.w_ff, W.w_down):
                if dn is not None:
                    n += dn.w.numel() * dn.w.element_size()
            if W.a2 is not None:
                n += W.a2.numel() * 4
        return n

    # ------------------------------------------------------------------ loading
    @classmethod
    def load(cls, cfg: GirulornConfig, get, device="cpu", dtype=None) -> "GirulornModel":
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

        for i, L in enumerate(cfg.layers):
            p, mx = f"l{i}.mix.", L.mixer
            kw = {}
            if L.type == "attention":
                H, G, dk, dv = mx.heads, mx.kv_heads, mx.dim, mx.vdim
                parts = [("q", t(p + "q", (H * dk, C)))]
                if mx.kv_from is None:
                    parts += [("k", t(p + "k", (G * dk, C))), ("v", t(p + "v", (G * dv, C)))]
                    kw["k_norm"] = f32(p + "k.norm", (dk,))
                parts.append(("g", t(p + "g", (H, C))))
                w_o = along_k([t(p + "o", (C, H * dv))])
                kw.update(q_norm=f32(p + "q.norm", (dk,)), sink=f32(p + "sink", (H,)),
                          bias=HY.log_bucket_table(t(p + "rel", (mx.bias_rows, H)), mx.bias_max).to(dev))
            else:
                H, dk, dv, r = mx.heads, mx.dim, mx.vdim, mx.rank
                parts = [("q", t(p + "q", (H * dk, C))), ("k", t(p + "k", (H * dk, C))), ("v", t(p + "v", (H * dv, C))),
                         ("g", t(p + "g", (H * dv, C))), ("a1", t(p + "a1", (r, C)))]
                w_o = along_k([t(p + "o", (C, H * dv))])
                kw.update(a2=t(p + "a2", (H * dk, r)).t().contiguous().to(dev), a2_b=f32(p + "a2.b", (H * dk,)),
                          mix_norm=f32(p + "norm", (dv,)))
            w_in, cols, n_in = stack(parts)
            f, q = L.mlp, f"l{i}.mlp."
            if f is not None:
                fparts = [("router", t(q + "router", (f.experts, C)))]
                outs = []
                if f.shared_ff:
                    fparts += [("sgate", t(q + "shared.gate", (f.shared_ff, C))),
                               ("sup", t(q + "shared.up", (f.shared_ff, C)))]
                    outs.append(t(q + "shared.down", (C, f.shared_ff)))
                fparts += [("egate", torch.cat([t(f"{q}e{e}.gate", (f.ff, C)) for e in range(f.experts)], 0)),
                           ("eup", torch.cat([t(f"{q}e{e}.up", (f.ff, C)) for e in range(f.experts)], 0))]
                outs += [t(f"{q}e{e}.down", (C, f.ff)) for e in range(f.experts)]
                w_ff, ff_cols, n_ff = stack(fparts)
                w_down = along_k(outs)
                kw.update(norm2=f32(f"l{i}.norm2", (C,)), w_ff=Dense(w_ff, None, dev, md),
                          w_down=Dense(w_down, None, dev, md), ff_cols=ff_cols, n_ff=n_ff, k_down=w_down.shape[1],
                          router_b=f32(q + "router.b", (f.experts,)))
            m.weights[i] = GirulornWeights(norm1=f32(f"l{i}.norm1", (C,)), w_in=Dense(w_in, None, dev, md),
                                           w_o=Dense(w_o, None, dev, md), cols=cols, n_in=n_in, k_o=w_o.shape[1], **kw)
        m.embed = t("embed", (cfg.vocab, C)).to(md).contiguous().to(dev)
        m.final_norm = f32("final.norm", (C,))
        m.head = Dense(t("head", (cfg.vocab, C)), None, dev, md)
        return m

    # ------------------------------------------------------------------ forward
    def forward(self, fb, cache, ws: GirulornWorkspace) -> torch.Tensor:
        cfg = self.cfg
        T, C, eps = fb.T, cfg.hidden, cfg.rms_eps
        if T > ws.max_tokens:
            raise ValueError(f"step of {T} tokens, workspace holds {ws.max_tokens}")
        b16 = self.dtype != torch.float32
        rag = HY.Ragged(fb)
        x = ws.x[:T]
        hin = ws.hin[:T] if b16 else x  # what the GEMMs read: the residual itself, rounded in bf16 mode
        x16 = hin if b16 else None
        HY.embed_rows(self.embed, fb.tokens, x, out16=x16)
        if fb.embed_rows:
            for r0, e in fb.embed_rows:
                x[r0:r0 + e.shape[0]].copy_(e)
            if b16:
                hin.copy_(x)
        o = ws.o[:T]
        for li, L in enumerate(cfg.layers):
            if fb.stop_layer is not None and li >= fb.stop_layer:
                break
            W = self.weights[li]
            y = ws.y[:T * W.n_in].view(T, W.n_in)
            W.w_in.into(hin, y)
            cat = ws.cat[:T * W.k_o].view(T, W.k_o)
            if L.type == "attention":
                own = li if L.mixer.kv_from is None else L.mixer.kv_from
                self._attention(L.mixer, W, y, fb, rag, cache.layer(own)[0], ws, cat, eps)
            else:
                self._gla(L.mixer, W, y, rag, cache.layer(li)[1], ws, cat, eps)
            W.w_o.into(cat, o)
            HY.norm_add(o, W.norm1, eps, x, x16)
            f = L.mlp
            if f is not None:
                c = W.ff_cols
                y = ws.y[:T * W.n_ff].view(T, W.n_ff)
                W.w_ff.into(hin, y)
                cat = ws.cat[:T * W.k_down].view(T, W.k_down)
                k0 = 0
                if f.shared_ff:
                    Fs = f.shared_ff
                    HY.glu(y[:, c["sgate"]:c["sgate"] + Fs], y[:, c["sup"]:c["sup"] + Fs], None, None, cat[:, :Fs])
                    k0 = Fs
                E = f.experts
                rw = ws.route[:T * E].view(T, E)
                HY.moe_route(y[:, c["router"]:c["router"] + E], f.top, 1.0, rw, 0.0, bias=W.router_b)
                HY.glu(y[:, c["egate"]:c["egate"] + E * f.ff], y[:, c["eup"]:c["eup"] + E * f.ff], None, None,
                       cat[:, k0:k0 + E * f.ff], scale=rw, group=f.ff)
                W.w_down.into(cat, o)
                HY.norm_add(o, W.norm2, eps, x, x16)
        if fb.stop_layer is not None:
            return x
        S = fb.logits_idx.numel()
        if S > ws.logits_rows:
            raise ValueError(f"{S} logit rows asked, workspace holds {ws.logits_rows}")
        hs = ws.hs[:S]
        HY.offset_rmsnorm(x, self.final_norm, eps, out32=None if b16 else hs, out16=hs if b16 else None,
                          rows=fb.logits_idx, offset=0.0)
        if fb.want_hidden or fb.keep_hidden:
            if fb.want_hidden:
                return hs.float()
            self.last_hidden = hs.float()
        return self.head.into(hs, ws.logits[:S])

    def _attention(self, a: BiasAttnCfg, W, y, fb, rag, kv, ws, cat, eps):
        T = y.shape[0]
        H, G, dk, dv = a.heads, a.kv_heads, a.dim, a.vdim
        c = W.cols
        q = ws.q[:T * H * dk].view(T, H * dk)
        own = a.kv_from is None
        HY.rope_norm_append(y[:, c["q"]:c["q"] + H * dk], y[:, c["k"]:c["k"] + G * dk] if own else None,
                            y[:, c["v"]:c["v"] + G * dv] if own else None, fb.positions, H, G, dk, dv, 0, 10000.0, True,
                            eps, q, kv[0] if own else None, kv[1] if own else None, fb.slots, q_weight=W.q_norm,
                            k_weight=W.k_norm, q_temp=(a.temp_coef, a.temp_every) if a.temp_coef else None)
        HY.masked_attention(q, kv[0], kv[1], rag, H, G, dk, dv, a.scale, cat[:, :H * dv], sink=W.sink, bias=W.bias,
                            gate=y[:, c["g"]:c["g"] + H], workspace=(ws.part_ml, ws.part_o))

    def _gla(self, g: GlaCfg, W, y, rag, state, ws, cat, eps):
        T = y.shape[0]
        H, dk, dv = g.heads, g.dim, g.vdim
        c = W.cols
        nk, nv = H * dk, H * dv
        decay = ws.decay[:T * nk].view(T, nk)  # second projection (fp32: its logits never see 16 bits), bias, decay
        HY.channel_decay(y[:, c["a1"]:c["a1"] + g.rank], W.a2_b, g.tau, decay, proj=W.a2)
        o = ws.scan[:T * nv].view(T, nv)
        HY.state_scan(y[:, c["k"]:c["k"] + nk], y[:, c["q"]:c["q"] + nk], y[:, c["v"]:c["v"] + nv], decay, None, None,
                      state, rag, o, H, H, dk, dv, delta=False, channel=True, q_scale=dk ** -0.5)
        HY.gated_group_norm(o, y[:, c["g"]:c["g"] + nv], W.mix_norm, eps, dv, cat[:, :nv], gate_first=False)


# ------------------------------------------------------------------------------------------------ sources
def is_girulorn_dir(path: str) -> bool:
    f = os.path.join(path, "config.json")
    if not (os.path.isdir(path) and os.path.isfile(f)):
        return False
    try:
        with open(f) as fh:
            return json.load(fh).get("architecture") == ARCH
    except (OSError, ValueError):
        return False


def dir_source(model_dir: str):
    """(GirulornConfig, get) of a directory holding config.json and model.safetensors."""
    from .vosotar import tensor_getter
    get = tensor_getter(model_dir)

    def shapes(name):
        a = get(name)
        if a is None:
            raise KeyError(f"checkpoint has no tensor {name!r}")
        return tuple(a.shape)
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = GirulornConfig.from_json(json.load(f), os.path.basename(os.path.normpath(model_dir)), shapes)
    return cfg, get


def tensor_shapes(cfg: GirulornConfig) -> dict:
    """name -> shape of every checkpoint tensor of a configuration."""
    C = cfg.hidden
    s = {"embed": (cfg.vocab, C), "final.norm": (C,), "head": (cfg.vocab, C)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.mix.", L.mixer
        s[f"l{i}.norm1"] = (C,)
        if L.type == "attention":
            s.update({p + "q": (m.heads * m.dim, C), p + "q.norm": (m.dim,), p + "rel": (m.bias_rows, m.heads),
                      p + "sink": (m.heads,), p + "g": (m.heads, C), p + "o": (C, m.heads * m.vdim)})
            if m.kv_from is None:
                s.update({p + "k": (m.kv_heads * m.dim, C), p + "v": (m.kv_heads * m.vdim, C), p + "k.norm": (m.dim,)})
        else:
            s.update({p + "q": (m.heads * m.dim, C), p + "k": (m.heads * m.dim, C), p + "v": (m.heads * m.vdim, C),
                      p + "g": (m.heads * m.vdim, C), p + "o": (C, m.heads * m.vdim), p + "norm": (m.vdim,),
                      p + "a1": (m.rank, C), p + "a2": (m.heads * m.dim, m.rank), p + "a2.b": (m.heads * m.dim,)})
        f, q = L.mlp, f"l{i}.mlp."
        if f is not None:
            s[f"l{i}.norm2"] = (C,)
            for e in range(f.experts):
                s.update({f"{q}e{e}.gate": (f.ff, C), f"{q}e{e}.up": (f.ff, C), f"{q}e{e}.down": (C, f.ff)})
            s.update({q + "router": (f.experts, C), q + "router.b": (f.experts,)})
            if f.shared_ff:
                s.update({q + "shared.gate": (f.shared_ff, C), q + "shared.up": (f.shared_ff, C),
                          q + "shared.down": (C, f.shared_ff)})
    return s


def synthetic_source(cfg: GirulornConfig, seed: int = 0):
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
            if leaf in ("norm1", "norm2", "norm") or name == "final.norm":
                a = 1.0 + 0.1 * torch.randn(s, generator=g)
            elif leaf in ("rel", "sink"):
                a = torch.randn(s, generator=g)
            elif name.endswith("a2.b"):
                a = 2.0 + torch.randn(s, generator=g)  # decays near one, as a trained layer keeps them
            elif leaf == "b":
                a = 0.5 * torch.randn(s, generator=g)
            elif leaf == "router":
                a = 2.0 * torch.randn(s, generator=g) * (s[-1] ** -0.5)
            else:
                a = torch.randn(s, generator=g) * (s[-1] ** -0.5)
            made[name] = a.to(torch.bfloat16)
        return made[name]
    get.names = order
    return get


def save_checkpoint(cfg: GirulornConfig, get, model_dir: str) -> None:
    """Write config.json + model.safetensors (bf16) of `get`'s tensors: the layout `dir_source` reads."""
    from safetensors.torch import save_file
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: get(k).contiguous() for k in get.names}, os.path.join(model_dir, "model.safetensors"))


def load_dir(model_dir: str, device="cpu", dtype=None) -> GirulornModel:
    cfg, get = dir_source(model_dir)
    return GirulornModel.load(cfg, get, device, dtype)
