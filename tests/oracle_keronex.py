"""Plain float64 whole-sequence oracle of the Keronex decoder, one function per mechanism, written from the model's
equations and sharing no code with the package. `forward(config dict, get, tokens)` -> logits [T, vocab]; `get(name)`
returns a checkpoint tensor. Everything is recomputed from position 0 for every call: no cache, no state."""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w.to(F64))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def pair_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every position: the extra last row at position 0."""
    rows = [buckets]
    for p in range(1, len(tokens)):
        rows.append((tokens[p - 1] * mul_prev + tokens[p] * mul_cur) % buckets)
    return rows


def embedding(d, get, tokens):
    e = d.get("embedding") or {}
    x = get("embed").to(F64)[tokens] * e.get("scale", 1.0)
    bg = e.get("bigram")
    if bg:
        x = x + get("bigram").to(F64)[pair_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])]
    return x


def rotate_halves(x, dims, base):
    """x [T, heads, d]: position p turns the pair (x[i], x[i + dims / 2]) by p * base^(-2 i / dims)."""
    if not dims:
        return x
    T, n2 = x.shape[0], dims // 2
    out = x.clone()
    for i in range(n2):
        ang = torch.arange(T, dtype=F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = x[..., i], x[..., i + n2]
        out[..., i] = a * c - b * s
        out[..., i + n2] = b * c + a * s
    return out


def softmax_map(q, k, v, scale):
    """One causal softmax attention: q, k [T, d], v [T, e]."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        s = (k[:i + 1] @ q[i]) * scale
        w = torch.exp(s - s.max())
        out[i] = (w / w.sum()) @ v[:i + 1]
    return out


def diff_lambda(m, get, p):
    a = (get(p + "lq1").to(F64) * get(p + "lk1").to(F64)).sum()
    b = (get(p + "lq2").to(F64) * get(p + "lk2").to(F64)).sum()
    return float(torch.exp(a) - torch.exp(b)) + m["diff"]


def differential_attention(q, k, v, scale, lam, diff, eps):
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, e]: per head unit_rms(map1 - lam map2) (1 - diff), [T, H, e]."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        a1 = softmax_map(q[:, h, 0], k[:, g, 0], v[:, g], scale)
        a2 = softmax_map(q[:, h, 1], k[:, g, 1], v[:, g], scale)
        out[:, h] = unit_rms(a1 - lam * a2, eps) * (1.0 - diff)
    return out


def attention_mixer(m, get, p, h, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    q = (h @ get(p + "q").to(F64).T).reshape(T, 2 * H, d)
    k = (h @ get(p + "k").to(F64).T).reshape(T, 2 * G, d)
    v = (h @ get(p + "v").to(F64).T).reshape(T, G, e)
    q = rotate_halves(q, rot.get("dims", 0), rot.get("base", 1.0)).reshape(T, H, 2, d)
    k = rotate_halves(k, rot.get("dims", 0), rot.get("base", 1.0)).reshape(T, G, 2, d)
    o = differential_attention(q, k, v, m["scale"], diff_lambda(m, get, p), m["diff"], eps)
    return o.reshape(T, H * e) @ get(p + "o").to(F64).T


def retention(q, k, v, decay):
    """q, k [T, H, d], v [T, H, e], decay [H]: S <- decay S + k v^T, o = S^T q."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F64)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = (S * q[t][:, :, None]).sum(1)
    return out


def retention_mixer(m, get, p, h, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    q = rotate_halves((h @ get(p + "q").to(F64).T).reshape(T, H, d), rot.get("dims", 0), rot.get("base", 1.0))
    k = rotate_halves((h @ get(p + "k").to(F64).T).reshape(T, H, d), rot.get("dims", 0), rot.get("base", 1.0))
    v = (h @ get(p + "v").to(F64).T).reshape(T, H, e)
    o = retention(q, k * d ** -0.5, v, torch.tensor(m["decay"], dtype=F64))
    g = h @ get(p + "g").to(F64).T
    return (unit_rms(o, eps).reshape(T, H * e) * g * torch.sigmoid(g)) @ get(p + "o").to(F64).T


def short_conv_silu(x, w):
    """x [T, C], w [C, taps] (last column: the current token); zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                y[t] += w[:, j] * x[src]
    return y * torch.sigmoid(y)


def channel_delta_rule(q, k, v, beta, g):
    """q, k, g [T, H, d], v [T, H, e], beta [T, H]: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F64)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for t in range(T):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - (S * k[t][:, :, None]).sum(1))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = (S * q[t][:, :, None]).sum(1)
    return out


def channel_delta_mixer(m, get, p, h, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    G = m.get("kv_heads", H)
    w = lambda n: get(p + n).to(F64)  # noqa: E731
    q = short_conv_silu(h @ w("q").T, w("q.conv")).reshape(T, G, d)
    k = short_conv_silu(h @ w("k").T, w("k.conv")).reshape(T, G, d)
    v = short_conv_silu(h @ w("v").T, w("v.conv")).reshape(T, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1)
    beta = torch.sigmoid(h @ w("b").T)
    z = ((h @ w("a1").T) @ w("a2").T + w("dt_bias")).reshape(T, H, d)
    g = torch.exp(-torch.exp(w("A_log"))[None, :, None] * torch.log1p(torch.exp(z)))
    o = unit_rms(channel_delta_rule(q, k, v, beta, g), eps) * w("norm")
    gate = torch.sigmoid((h @ w("g1").T) @ w("g2").T)
    return (o.reshape(T, H * e) * gate) @ w("o").T


def dense_ff(get, p, h):
    w = lambda n: get(p + n).to(F64)  # noqa: E731
    return (gelu_tanh(h @ w("gate").T) * (h @ w("up").T)) @ w("down").T


def squared_relu_expert(get, p, x):
    return (torch.relu(x @ get(p + "up").to(F64).T) ** 2) @ get(p + "down").to(F64).T


def route(scores, top):
    """scores [E] -> [(expert, weight)]: the `top` largest sigmoid scores, kept as they are."""
    order = sorted(range(len(scores)), key=lambda e: (-float(scores[e]), e))[:top]
    return [(e, scores[e]) for e in order]


def mixture(f, get, p, h):
    out = torch.zeros_like(h)
    s = torch.sigmoid(h @ get(p + "router").to(F64).T)
    for t in range(h.shape[0]):
        for e, w in route(s[t], f["router"]["top"]):
            out[t] += squared_relu_expert(get, f"{p}e{e}.", w * h[t])  # the weight multiplies the expert's INPUT
    if f.get("shared"):
        out = out + squared_relu_expert(get, p + "shared.", h)
    return out


def hyper_read(xs, w_in):
    return sum(w_in[s] * xs[s] for s in range(len(xs)))


def hyper_write(xs, y, mix, w_out):
    n = len(xs)
    return [sum(mix[s, t] * xs[s] for s in range(n)) + w_out[t] * y for t in range(n)]


MIXERS = {"attention": attention_mixer, "retention": retention_mixer, "channel_delta": channel_delta_mixer}


def forward(d, get, tokens, layers=None):
    """logits [T, vocab]; `layers` (a list) receives the sum of the streams after every layer."""
    eps = d["norm"]["eps"]
    x = embedding(d, get, list(tokens))
    S = d.get("streams")
    xs = [x.clone() for _ in range(S or 1)]
    for i, L in enumerate(d["layers"]):
        j = L.get("weights_of", i)
        subs = [("1", lambda h, L=L, j=j: MIXERS[L["type"]](L["mixer"], get, f"l{j}.mix.", h, eps))]
        f = L.get("mlp")
        if f is not None:
            fn = dense_ff if f["kind"] == "dense" else lambda g_, p, h, f=f: mixture(f, g_, p, h)
            subs.append(("2", lambda h, fn=fn, j=j: fn(get, f"l{j}.mlp.", h)))
        for n, sub in subs:
            w = get(f"l{j}.norm{n}")
            if S is None:
                xs = [xs[0] + sub(offset_norm(xs[0], w, eps))]
                continue
            hc = lambda k: get(f"l{j}.hc{n}.{k}").to(F64)  # noqa: E731
            y = sub(offset_norm(hyper_read(xs, hc("in")), w, eps))
            xs = hyper_write(xs, y, hc("mix"), hc("out"))
        if layers is not None:
            layers.append(sum(xs))
    return offset_norm(sum(xs), get("final.norm"), eps) @ get("head").to(F64).T
