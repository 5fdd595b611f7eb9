"""A slow float64 whole-sequence oracle of the Girulorn decoder, one function per mechanism. It takes the configuration
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


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * d(w)


def silu(z):
    return z * torch.sigmoid(z)


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance-bias table for distance n >= 0: the first half of the rows are exact distances, the other
    half spread logarithmically up to `far`; everything beyond lands in the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def query_temperature(pos: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((pos + 1) // every + 1)


def sink_bias_attention(q, k, v, scale, rel, far, sink):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv]; rel [rows, H] distance-bias table, sink [H]. Token i sees every j <= i;
    score = scale q.k + rel[bucket(i - j), h]; the softmax denominator has one more term exp(sink_h) without a value."""
    T, H, _ = q.shape
    G = k.shape[1]
    rows = rel.shape[0]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    bk = torch.tensor([distance_bucket(n, rows, far) for n in range(T)])
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[:i + 1, g] @ q[i, h]) * scale
            s = s + d(rel)[bk[i - torch.arange(i + 1)], h]
            m = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * v[:i + 1, g]).sum(0) / (math.exp(float(sink[h]) - m) + e.sum())
    return out


def attention_keys_values(h, m, get, p, eps):
    """Keys (normed, as the cache keeps them) and values of an attention layer that owns them."""
    T = h.shape[0]
    G, dk, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = rms_norm((h @ d(get(p + "k")).T).reshape(T, G, dk), get(p + "k.norm"), eps)
    v = (h @ d(get(p + "v")).T).reshape(T, G, dv)
    return k, v


def attention_mixer(h, m, get, p, eps, kv):
    """h [T, C]; m the layer's mixer dictionary; kv = (keys, values) of this layer or of the layer it borrows from."""
    T = h.shape[0]
    H, dk = m["heads"], m["dim"]
    q = rms_norm((h @ d(get(p + "q")).T).reshape(T, H, dk), get(p + "q.norm"), eps)
    qt = m.get("q_temp")
    if qt:
        f = torch.tensor([query_temperature(i, float(qt["coef"]), int(qt["every"])) for i in range(T)], dtype=F64)
        q = q * f[:, None, None]
    o = sink_bias_attention(q, kv[0], kv[1], float(m["scale"]), get(p + "rel"), float(m["bias_max"]), d(get(p + "sink")))
    o = o * torch.sigmoid(h @ d(get(p + "g")).T)[:, :, None]
    return o.reshape(T, -1) @ d(get(p + "o")).T


def channel_decay_recurrence(q, k, v, alpha):
    """q, k, alpha [T, H, dk], v [T, H, dv]: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, S_0 = 0."""
    T, H, dk = q.shape
    S = torch.zeros(H, dk, v.shape[2], dtype=F64)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def gla_mixer(h, m, get, p, eps):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ d(get(p + "q")).T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ d(get(p + "k")).T).reshape(T, H, dk)
    v = (h @ d(get(p + "v")).T).reshape(T, H, dv)
    z = (h @ d(get(p + "a1")).T) @ d(get(p + "a2")).T + d(get(p + "a2.b"))
    alpha = torch.sigmoid(z).pow(1.0 / float(m["tau"])).reshape(T, H, dk)
    o = rms_norm(channel_decay_recurrence(q, k, v, alpha), get(p + "norm"), eps).reshape(T, H * dv)
    return (o * silu(h @ d(get(p + "g")).T)) @ d(get(p + "o")).T


def glu_expert(h, get, p):
    return (silu(h @ d(get(p + "gate")).T) * (h @ d(get(p + "up")).T)) @ d(get(p + "down")).T


def expert_mixture(h, f, get, p):
    """The `top` experts of largest router logit, weighted by the softmax over those logits alone, plus the shared
    expert."""
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ d(get(p + "router")).T + d(get(p + "router.b"))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        idx = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, idx], 0)
        for wi, e in zip(w, idx):
            out[t] += wi * glu_expert(h[t:t + 1], get, f"{p}e{e}.")[0]
    if f.get("shared"):
        out = out + glu_expert(h, get, p + "shared.")
    return out


def forward(cfg: dict, get, tokens, layers_out: list | None = None):
    """Logits [T, vocab] (float64) of one whole sequence; `layers_out` collects the residual after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = d(get("embed"))[torch.as_tensor(tokens).long()]
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        if L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = attention_keys_values(x, m, get, p, eps)
                src = i
            y = attention_mixer(x, m, get, p, eps, kv[src])
        elif L["type"] == "gla":
            y = gla_mixer(x, m, get, p, eps)
        else:
            raise ValueError(L["type"])
        x = x + rms_norm(y, get(f"l{i}.norm1"), eps)
        if L.get("mlp") is not None:
            x = x + rms_norm(expert_mixture(x, L["mlp"], get, f"l{i}.mlp."), get(f"l{i}.norm2"), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, get("final.norm"), eps) @ d(get("head")).T
