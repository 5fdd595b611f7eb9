"""Ops of hybrid decoders that mix paged softmax attention with recurrent layers whose state is carried per sequence:

* `embed_rows`, `offset_rmsnorm`, `norm_add`: an fp32 residual from a 16-bit table; an RMS norm whose weight is
  stored around an offset (x / rms * (offset + w)); the same norm applied to a sublayer's OUTPUT and added to the
  residual (x += y / rms(y) * (offset + w)), with the 16-bit copy of the new residual the next GEMM reads;
* `rope_norm_append`: rotary positions on neighbouring pairs of the first `rot_dims` numbers of each query / key
  head, an optional unit-RMS norm of every head after the rotation (with optional per-channel weights), an optional
  position-dependent query temperature, and the append of keys and values to paged pools;
* `masked_attention`: causal attention over the paged pools whose visible range starts at a chunk border
  (`chunk`), `window` keys back, or at position 0, with an optional sink (one extra term exp(0), or exp(s_h) with a
  learned s_h per head, in the softmax denominator that carries no value), an optional additive bias that depends on
  the distance between query and key (`log_bucket_table`) and an optional sigmoid gate per token and head;
* `causal_conv`: a per-channel causal convolution over time (optional bias and SiLU) whose last taps-1 inputs are
  carried per sequence;
* `unit_norm_heads`, `scan_coefs`, `channel_decay`, `state_scan`: the pieces of a linear recurrence
  S <- a S + k u^T, o = S^T q per head (S is [N, P], fp32, one per sequence and head, stored column-major). With
  `delta` the written value is u = c (v - S^T k) after the decay (gated delta rule), otherwise u = c v with an
  optional skip D v on the output (state-space duality form); the decay a is one number per head or, for gated
  linear attention, one per key channel (S <- diag(a) S + k v^T, a = sigmoid(z)^(1/tau));
* `gated_group_norm`: unit-RMS norm over groups of columns, a weight, and a SiLU gate before or after the norm;
* `glu`: silu(a + bias) * (b + bias) with an optional per-row, per-column-group factor (routing weights of experts
  evaluated side by side, or the sigmoid gate of a shared expert);
* `moe_route`: softmax over experts (optional logit bias), the `top` largest, renormalised and scaled, as a dense
  [T, E] weight matrix (with eps = 0 and scale = 1 that is the softmax over the chosen logits alone); or, in the
  `sigmoid` mode, the chosen experts' sigmoid scores as they are;
* `embed_pair`: a scaled token embedding plus a row of a second table picked by a hash of (previous token, token); the
  previous token is carried per sequence;
* `hyper_step`: a residual kept as several streams: the streams are mixed among themselves and take a sublayer's
  output with one weight each, and the next sublayer's input is a weighted sum of the streams, normed;
* `rope_rows`: rotary positions in place, on neighbouring pairs or on the pairs (i, i + rot_dims / 2);
* `diff_group_norm`: unit-RMS norm over groups of columns of a - lam * b (two attention maps over the same values).

Every function runs the HIP kernels of csrc/kernels/hybrid/ on GPU tensors and a plain fp32 PyTorch form on CPU
tensors (the plumbing path of GPU-less environments). Positions, angles, scores, softmax, norms, routing, decays,
states and the residual are fp32 in both; 16-bit tensors appear only as GEMM operands and in the paged pools.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from .. import _native as N
from .latent import Ragged, _is16  # noqa: F401  (Ragged: the step layout shared with the latent ops)


def _f32c(t: torch.Tensor, what: str):
    if t.dtype != torch.float32 or t.stride(-1) != 1:
        raise TypeError(f"{what}: fp32 rows with a contiguous last axis expected")


# ------------------------------------------------------------------------------------------------ embedding, norm
def embed_rows(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
               out16: torch.Tensor | None = None):
    """out[t] (=|+=) table[tokens[t]]; table fp32 or bf16 [V, C], out fp32 [T, C]; `out16` (bf16 [T, C]) also receives
    the result, rounded (the operand of a GEMM that reads the residual itself)."""
    T, C = out.shape
    if T == 0:
        return out
    if not out.is_cuda:
        rows = table[tokens.long()].float()
        out.add_(rows) if accumulate else out.copy_(rows)
        if out16 is not None:
            out16.copy_(out)
        return out
    N.kcall("mxh_embed_rows", table.data_ptr(), _is16(table), table.shape[0], tokens.data_ptr(), out.data_ptr(),
            out.stride(0), int(accumulate), N.ptr(out16), out16.stride(0) if out16 is not None else 0, T, C,
            N.stream_ptr())
    return out


def offset_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, out32: torch.Tensor | None = None,
                   out16: torch.Tensor | None = None, rows: torch.Tensor | None = None, offset: float = 1.0):
    """y = x / sqrt(mean(x^2) + eps) * (offset + w) for fp32 rows, written as fp32 and / or bf16. `rows` (int32)
    picks the rows of x to norm: output row i comes from x[rows[i]]."""
    M = int(rows.numel()) if rows is not None else x.shape[0]
    C = x.shape[1]
    if M == 0:
        return
    if not x.is_cuda:
        xs = x[rows.long()] if rows is not None else x
        y = xs * torch.rsqrt(xs.pow(2).mean(-1, keepdim=True) + eps) * (offset + w.float())
        if out32 is not None:
            out32.copy_(y)
        if out16 is not None:
            out16.copy_(y)
        return
    _f32c(x, "offset_rmsnorm")
    N.kcall("mxh_offset_norm", x.data_ptr(), x.stride(0), N.ptr(rows), w.data_ptr(), float(offset), float(eps),
            N.ptr(out32), out32.stride(0) if out32 is not None else 0, N.ptr(out16),
            out16.stride(0) if out16 is not None else 0, M, C, N.stream_ptr())


def norm_add(y: torch.Tensor, w: torch.Tensor, eps: float, x: torch.Tensor, out16: torch.Tensor | None = None,
             offset: float = 0.0):
    """x += y / sqrt(mean(y^2) + eps) * (offset + w) for fp32 rows y, x [T, C] (the norm sits on a sublayer's output,
    the residual takes the normed value); `out16` (bf16 [T, C]) receives the new residual rounded, for the GEMM that
    reads it next."""
    T, C = y.shape
    if T == 0:
        return x
    if not y.is_cuda:
        x.add_(y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * (offset + w.float()))
        if out16 is not None:
            out16.copy_(x)
        return x
    _f32c(y, "norm_add")
    _f32c(x, "norm_add")
    N.kcall("mxh_norm_add", y.data_ptr(), y.stride(0), w.data_ptr(), float(offset), float(eps), x.data_ptr(),
            x.stride(0), N.ptr(out16), out16.stride(0) if out16 is not None else 0, T, C, N.stream_ptr())
    return x


def embed_pair(table: torch.Tensor, pair: torch.Tensor | None, tokens: torch.Tensor, rag: "Ragged",
               last_token: torch.Tensor | None, scale: float, mul_prev: int, mul_cur: int, buckets: int,
               out: torch.Tensor, copies: int = 1):
    """out[t] = scale * table[tokens[t]] + pair[(prev_t * mul_prev + tokens[t] * mul_cur) mod buckets], written
    `copies` times side by side (out fp32 [T, copies * C]). prev_t is the token before row t in its sequence: the row
    above inside a chunk, `last_token[slot]` (int32 [slots]) for a chunk's first row, and for position 0 there is none:
    that row takes pair[buckets], the table's last row. Each sequence's last token of the step is left in
    `last_token[slot]`. pair = None: the scaled embedding alone. Tables are fp32 or bf16."""
    T = tokens.numel()
    C = table.shape[1]
    if T == 0:
        return out
    if out.shape != (T, copies * C) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError("embed_pair: out is a contiguous fp32 [T, copies * C]")
    if pair is not None and (pair.shape != (buckets + 1, C) or last_token is None or last_token.dtype != torch.int32):
        raise ValueError("embed_pair: the pair table has buckets + 1 rows; previous tokens are int32 per slot")
    if not out.is_cuda:
        tk = tokens.long()
        x = table[tk].float() * scale
        if pair is not None:
            st, pos = rag.state.tolist(), rag.positions.tolist()
            for r0, n, si in rag.host_segments():
                slot = st[si]
                prev = torch.empty(n, dtype=torch.long)
                prev[1:] = tk[r0:r0 + n - 1]
                first_none = pos[r0] == 0
                prev[0] = 0 if (first_none or slot < 0) else int(last_token[slot])
                row = (prev * mul_prev + tk[r0:r0 + n] * mul_cur) % buckets
                if first_none:
                    row[0] = buckets
                x[r0:r0 + n] += pair[row].float()
                if slot >= 0:
                    last_token[slot] = int(tk[r0 + n - 1])
        out.copy_(x.repeat(1, copies))
        return out
    if pair is not None and _is16(pair) != _is16(table):
        raise TypeError("embed_pair: both tables share one dtype")
    N.kcall("mxh_embed_pair", table.data_ptr(), N.ptr(pair), _is16(table), table.shape[0], tokens.data_ptr(),
            rag.state.data_ptr(), rag.positions.data_ptr(), rag.n_dec, N.ptr(rag.pf_cu), rag.n_pf, N.ptr(last_token),
            float(scale), int(mul_prev), int(mul_cur), int(buckets), out.data_ptr(), int(copies), T, C, N.stream_ptr())
    return out


HYPER_MAX_STREAMS = 32  # (up to 8 streams keep a column's values and the coefficients in registers)


def hyper_step(xs: torch.Tensor, y: torch.Tensor | None, mix: torch.Tensor | None, out_w: torch.Tensor | None,
               in_w: torch.Tensor | None, norm_w: torch.Tensor | None, eps: float, h32: torch.Tensor | None = None,
               h16: torch.Tensor | None = None, total: torch.Tensor | None = None, offset: float = 1.0):
    """A residual of S streams xs fp32 [T, S * C] (stream s of a row in columns [s C, (s + 1) C)). With y (fp32 [T, C],
    a sublayer's output): all streams at once from the old ones, x_t <- sum_s mix[s, t] x_s + out_w[t] y (mix fp32
    [S, S] indexed [from, to], out_w fp32 [S]). With in_w (fp32 [S]): u = sum_s in_w[s] x_s of the updated streams and
    h = u / sqrt(mean(u^2) + eps) * (offset + norm_w), written as fp32 (`h32`) and / or bf16 (`h16`): the input of the
    next sublayer. `total` (fp32 [T, C]) receives the sum of the updated streams. One pass over the row."""
    T = xs.shape[0]
    if T == 0:
        return
    C = (y if y is not None else h32 if h32 is not None else h16 if h16 is not None else total).shape[1]
    S = xs.shape[1] // C
    if xs.shape[1] != S * C or S < 1 or S > HYPER_MAX_STREAMS:
        raise ValueError(f"hyper_step: 1 to {HYPER_MAX_STREAMS} streams of one width")
    if (y is None) != (mix is None) or (y is None) != (out_w is None) or (in_w is None) != (norm_w is None):
        raise ValueError("hyper_step: an update needs y, mix and out_w; a read needs in_w and norm_w")
    if not xs.is_cuda:
        X = xs.view(T, S, C)
        if y is not None:
            X.copy_(torch.einsum("st,nsc->ntc", mix.float(), X) + out_w.float()[None, :, None] * y.float()[:, None, :])
        if in_w is not None:
            u = torch.einsum("s,nsc->nc", in_w.float(), X)
            h = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * (offset + norm_w.float())
            if h32 is not None:
                h32.copy_(h)
            if h16 is not None:
                h16.copy_(h)
        if total is not None:
            total.copy_(X.sum(1))
        return
    _f32c(xs, "hyper_step")
    if not xs.is_contiguous() or (y is not None and (y.dtype != torch.float32 or y.stride(1) != 1)):
        raise TypeError("hyper_step: contiguous fp32 streams, fp32 rows of y")
    N.kcall("mxh_hyper_step", xs.data_ptr(), N.ptr(y), y.stride(0) if y is not None else 0, N.ptr(mix), N.ptr(out_w),
            N.ptr(in_w), N.ptr(norm_w), float(offset), float(eps), N.ptr(h32), h32.stride(0) if h32 is not None else 0,
            N.ptr(h16), h16.stride(0) if h16 is not None else 0, N.ptr(total),
            total.stride(0) if total is not None else 0, T, S, C, N.stream_ptr())


# ------------------------------------------------------------------------------------------------ attention
def log_bucket_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """Expands a bucketed distance-bias table rel [B, H] into one entry per distance and head: out [H, ceil(far) + 1]
    fp32 (a head's entries contiguous: neighbouring keys are neighbouring numbers) with out[h, n] = rel[bucket(n), h],
    bucket(n) = n for n < B/2, else min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(far / (B/2)) * (B - B/2))). Every
    distance >= far lands in the last bucket, so the last entry serves all of them (`masked_attention` clamps the
    distance to the table)."""
    B = rel.shape[0]
    half = B // 2
    if half < 1 or far <= half:
        raise ValueError("log_bucket_table: at least two rows, and the far distance lies beyond the exact half")
    n = torch.arange(int(math.ceil(far)) + 1, dtype=torch.float64)
    v = torch.log(n.clamp(min=half) / half) / math.log(far / half) * (B - half)
    v = torch.where((v - v.round()).abs() < 1e-9, v.round(), v)  # a whole number up to the rounding of the logarithms
    idx = torch.where(n < half, n, (half + v.floor()).clamp(max=B - 1)).long()
    return rel.float()[idx.to(rel.device)].t().contiguous()


def rope_norm_append(q_in: torch.Tensor, k_in: torch.Tensor, v_in: torch.Tensor, positions: torch.Tensor, H: int,
                     G: int, dk: int, dv: int, rot_dims: int, rot_base: float, norm: bool, eps: float,
                     q_out: torch.Tensor, kc: torch.Tensor | None, vc: torch.Tensor | None, slots: torch.Tensor,
                     q_weight: torch.Tensor | None = None, k_weight: torch.Tensor | None = None, q_temp=None,
                     half: bool = False, v_heads: int | None = None):
    """q_in [T, H*dk], k_in [T, G*dk], v_in [T, Gv*dv] (Gv = v_heads, G when not given: the value pool may hold fewer
    heads than the key pool): fp32 column slices of one projection output. Pair (2i, 2i+1), or with `half` the pair
    (i, i + rot_dims/2), of a head's first rot_dims numbers turns by positions[t] * rot_base^(-2i / rot_dims); with
    `norm` every query
    and key head is then divided by its root mean square (eps inside the root) and multiplied by q_weight / k_weight
    (fp32 [dk], shared by the heads) when given. `q_temp` = (coef, every) multiplies the query at position p by
    1 + coef * ln(floor((p + 1) / every) + 1). Queries go to q_out [T, H*dk] (fp32 or bf16), keys and values into the
    paged pools kc [blocks, bs, G*dk] / vc [blocks, bs, G*dv] at flat slot slots[t] (slot < 0: not stored). With
    k_in = None only the queries are made (a layer that reads another layer's keys and values)."""
    T = q_in.shape[0]
    if T == 0:
        return
    if rot_dims % 2 or rot_dims > dk:
        raise ValueError("rope_norm_append: rot_dims is even and at most the head size")
    Gv = G if v_heads is None else int(v_heads)
    if not q_in.is_cuda:
        def turn(x, n, w=None):
            x = _rope_ref(x.float().reshape(T, n, dk), positions, rot_dims, rot_base, half)
            if norm:
                x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
                if w is not None:
                    x = x * w.float()
            return x.reshape(T, n * dk)
        qn = turn(q_in, H, q_weight)
        if q_temp is not None:
            coef, every = float(q_temp[0]), int(q_temp[1])
            qn = qn * (1.0 + coef * torch.log((torch.div(positions + 1, every, rounding_mode="floor") + 1).float()))[:, None]
        q_out.copy_(qn)
        if k_in is None:
            return
        ok = slots >= 0
        kc.view(-1, G * dk)[slots[ok].long()] = turn(k_in, G, k_weight)[ok].to(kc.dtype)
        vc.view(-1, Gv * dv)[slots[ok].long()] = v_in.float()[ok].to(vc.dtype)
        return
    if (q_weight is not None or k_weight is not None) and not norm:
        raise ValueError("rope_norm_append: head weights belong to the head norm")
    if k_in is None:  # queries only: no key / value heads in the grid
        k_in = v_in = q_in
        kc = vc = q_out
        G = Gv = 0
    else:
        if kc.dtype != vc.dtype or not kc.is_contiguous() or not vc.is_contiguous():
            raise TypeError("rope_norm_append: contiguous key and value pools of one dtype")
    for t_ in (q_in, k_in, v_in):
        _f32c(t_, "rope_norm_append")
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 1)
    if every < 1:
        raise ValueError("rope_norm_append: the temperature steps every >= 1 positions")
    N.kcall("mxh_rope_norm_append", q_in.data_ptr(), k_in.data_ptr(), v_in.data_ptr(), q_in.stride(0),
            k_in.stride(0), v_in.stride(0), positions.data_ptr(), H, G, dk, dv, rot_dims, float(rot_base), int(norm),
            float(eps), q_out.data_ptr(), q_out.stride(0), _is16(q_out), kc.data_ptr(), vc.data_ptr(), _is16(kc),
            slots.data_ptr(), N.ptr(q_weight), N.ptr(k_weight), coef, every, int(half), Gv, T, N.stream_ptr())


def _rope_ref(x: torch.Tensor, positions: torch.Tensor, rot_dims: int, rot_base: float, half: bool) -> torch.Tensor:
    """x fp32 [T, n, d]: a copy whose first rot_dims numbers per head are turned by the rows' positions."""
    x = x.clone()
    if rot_dims:
        n2 = rot_dims // 2
        i = torch.arange(n2, dtype=torch.float32)
        a = positions.float()[:, None] * torch.exp(i * (-2.0 / rot_dims * math.log(rot_base)))[None, :]
        c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
        lo, hi = (slice(0, n2), slice(n2, rot_dims)) if half else (slice(0, rot_dims, 2), slice(1, rot_dims, 2))
        u, v = x[..., lo].clone(), x[..., hi].clone()
        x[..., lo] = u * c - v * s
        x[..., hi] = v * c + u * s
    return x


def rope_rows(x: torch.Tensor, positions: torch.Tensor, heads: int, dim: int, rot_dims: int, rot_base: float,
              half: bool = False, scale: float = 1.0, split: int | None = None, scale2: float = 1.0):
    """In place on fp32 x [T, heads*dim] (may be a column slice): rotary positions on the first rot_dims numbers of
    every head (pairs as in `rope_norm_append`), then the head times `scale`; heads from index `split` on take
    `scale2` (queries and keys side by side in one launch). For mixers that keep no keys per token."""
    T = x.shape[0]
    if T == 0:
        return x
    if rot_dims % 2 or rot_dims > dim:
        raise ValueError("rope_rows: rot_dims is even and at most the head size")
    split = heads if split is None else split
    if not x.is_cuda:
        v = _rope_ref(x.float().reshape(T, heads, dim), positions, rot_dims, rot_base, half)
        sc = torch.full((heads, 1), float(scale))
        sc[split:] = scale2
        x.copy_((v * sc).reshape(T, heads * dim))
        return x
    _f32c(x, "rope_rows")
    if dim > 512:
        raise ValueError("rope_rows: heads of up to 512 numbers")
    N.kcall("mxh_rope_rows", x.data_ptr(), x.stride(0), positions.data_ptr(), heads, dim, rot_dims, float(rot_base),
            int(half), float(scale), int(split), float(scale2), T, N.stream_ptr())
    return x


def _attn_ref(q, kc, vc, table, ctx, pos0, H, G, dk, dv, scale, chunk, window, sink, out, out_scale, sink_v=None,
              bias=None, gate=None, Gv=None):
    bs = kc.shape[1]
    nb = -(-ctx // bs)
    k = kc[table[:nb].long()].reshape(nb * bs, G, dk)[:ctx].float()
    Gv = G if Gv is None else Gv
    v = vc[table[:nb].long()].reshape(nb * bs, Gv, dv)[:ctx].float()
    if Gv != G:  # key head g reads value head g % Gv
        v = v[:, torch.arange(G) % Gv]
    n = q.shape[0]
    qh = q.float().reshape(n, H, dk)
    rep = H // G
    s = torch.einsum("nhd,jhd->hnj", qh, k.repeat_interleave(rep, 1)) * scale
    i = pos0 + torch.arange(n)[:, None]
    j = torch.arange(ctx)[None, :]
    lo = (i // chunk) * chunk if chunk else (i - window + 1).clamp(min=0) if window else torch.zeros_like(i)
    vis = (j <= i) & (j >= lo)
    if bias is not None:
        s = s + bias.float()[:, (i - j).clamp(0, bias.shape[1] - 1)]
    s = s.masked_fill(~vis[None], float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink:
        s0 = sink_v.float()[:, None, None] if sink_v is not None else torch.zeros(H, 1, 1)
        m = torch.maximum(m, s0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True) + (torch.exp(s0 - m) if sink else 0.0)
    o = torch.einsum("hnj,jhe->nhe", e / den, v.repeat_interleave(rep, 1))
    if gate is not None:
        o = o * torch.sigmoid(gate.float())[:, :, None]
    out.copy_((o.reshape(n, H * dv) * out_scale).to(out.dtype))


MFMA_MIN_ROWS = 16  # bf16 prompt chunks of at least this many rows take the matrix-core kernel (head sizes 64 / 128)
GEMM_MIN_ROWS = 64  # other prompt chunks of at least this many rows take the library-GEMM route (GPU)
GEMM_MAX_SCORES = 1 << 26  # fp32 scores of one sub-problem of that route
DECODE_WAVES = 4096  # decode rows: waves to aim for when splitting contexts into key partitions


def decode_part_len(n_dec: int, heads: int, visible: int) -> int:
    """Keys per partition of the decode rows: one wave walks a (row, head, partition), so few sequences with long
    visible ranges are split finely (down to one 64-key tile) and large batches coarsely."""
    want = max(1, DECODE_WAVES // max(1, n_dec * heads))
    per = -(-max(1, visible) // want)
    return max(64, -(-per // 64) * 64)


def _visible_blocks(p0: int, n: int, chunk: int, window: int, heads: int):
    """Sub-problems (first row position, end row position, first key position) of a chunk of n rows starting at
    position p0: rows of one mask chunk share their first key; every block's fp32 scores stay within
    GEMM_MAX_SCORES."""
    out = []
    if chunk:
        spans = [(max(p0, c * chunk), min(p0 + n, (c + 1) * chunk), c * chunk)
                 for c in range(p0 // chunk, (p0 + n - 1) // chunk + 1)]
    else:
        spans = [(p0, p0 + n, None)]
    for a, b, key0 in spans:
        k0 = key0 if key0 is not None else 0
        rows = max(GEMM_MIN_ROWS, GEMM_MAX_SCORES // max(1, heads * (b - k0)))
        for a2 in range(a, b, rows):
            b2 = min(b, a2 + rows)
            out.append((a2, b2, key0 if key0 is not None else max(0, a2 - window + 1) if window else 0))
    return out


def _attn_gemm_chunk(q, kc, vc, table, p0, n, H, G, dk, dv, scale, chunk, window, sink, out, out_scale, sink_v=None,
                     bias=None, gate=None, Gv=None, p32=False):
    """A long prompt chunk (rows q [n, H*dk] at positions p0 ..) as library GEMMs: per block of rows, the visible keys
    and values are gathered head-major from the pages, scores = Q K^T (fp32), masked sink softmax, out = P V (fp32).
    With `p32` and bf16 operands every softmax weight is written as two bf16 numbers (its rounding and the rest), side
    by side along K, and the values are stacked twice: the product sees the weights to 16 bits of mantissa."""
    from .dense import bmm_f32
    st = N.stream_ptr()
    md, dev, rep, bs = q.dtype, q.device, H // G, kc.shape[1]
    i16 = _is16(q)
    for a, b, key0 in _visible_blocks(p0, n, chunk, window, H):
        n2, nk = b - a, b - key0
        kh = torch.empty((G, nk, dk), dtype=md, device=dev)
        vh = torch.empty((G, nk, dv), dtype=md, device=dev)
        N.kcall("mxh_kv_gather", kc.data_ptr(), vc.data_ptr(), i16, bs, table.data_ptr(), key0, nk, G, dk, dv,
                kh.data_ptr(), vh.data_ptr(), G if Gv is None else Gv, st)
        qh = torch.empty((H, n2, dk), dtype=md, device=dev)
        qr = q[a - p0:]
        N.kcall("mxh_head_transpose", qr.data_ptr(), i16, qr.stride(0), dk, qh.data_ptr(), i16, dk, n2 * dk, n2, H, dk,
                1.0, None, 0, st)
        sc = bmm_f32(qh.view(G, rep * n2, dk), kh.transpose(1, 2))
        two = bool(p32 and i16)
        pw = torch.empty((G, rep * n2, 2 * nk if two else nk), dtype=md, device=dev)
        N.kcall("mxh_masked_softmax", sc.data_ptr(), pw.data_ptr(), i16, H * n2, n2, nk, a, key0, float(scale),
                int(chunk), int(window), int(sink), N.ptr(sink_v), N.ptr(bias), bias.shape[1] if bias is not None else 0,
                H, int(two), st)
        o = bmm_f32(pw, torch.cat([vh, vh], 1) if two else vh)
        orow = out[a - p0:]
        grow = gate[a - p0:] if gate is not None else None
        N.kcall("mxh_head_transpose", o.data_ptr(), 0, dv, n2 * dv, orow.data_ptr(), _is16(out), orow.stride(0), dv, n2,
                H, dv, float(out_scale), N.ptr(grow), grow.stride(0) if grow is not None else 0, st)


def masked_attention(q: torch.Tensor, kc: torch.Tensor, vc: torch.Tensor, rag: Ragged, H: int, G: int, dk: int, dv: int,
                     scale: float, out: torch.Tensor, chunk: int = 0, window: int = 0, sink=False,
                     out_scale: float = 1.0, workspace=None, bias: torch.Tensor | None = None,
                     gate: torch.Tensor | None = None, v_heads: int | None = None, p32: bool = False):
    """Causal attention of q [T, H*dk] over the paged pools (rope_norm_append's layout); query head h reads key
    head g = h // (H / G) and value head g % v_heads (v_heads = G when not given; fewer value heads than key heads:
    several attention maps over the same values). `p32`: softmax weights enter the value product with more than
    bf16's mantissa also in bf16 mode (the row kernels keep them in fp32 anyway; the matrix-core kernels and the GEMM
    route split each weight into two bf16 numbers, its rounding and the rounding of the rest). The row at position i
    sees j in [lo, i]: lo = (i // chunk) * chunk with `chunk`, max(0, i - window + 1) with `window`, else 0. `sink` = True adds exp(0) to the softmax denominator, an fp32 tensor
    [H] adds exp(sink[h]). `bias` (fp32 [H, L], contiguous) adds bias[h, min(i - j, L - 1)] to the scaled score.
    `gate` (fp32 [T, H], may be a column slice) multiplies head h's output of row t by sigmoid(gate[t, h]). out
    [T, H*dv] (may be a column slice; fp32 or bf16) receives out_scale times the result. q, pools and out share fp32
    or bf16 operands; scores, softmax and the accumulators are fp32.

    On the GPU decode rows and short chunks run the row kernel (one wave per row and head; decode rows split their
    visible keys into partitions merged through `workspace` = (fp32 [rows, 2], fp32 [rows, dv]), rows >= n_dec * H
    * partitions). bf16 tensors with head sizes of 64 or 128 run on the matrix cores: decode rows (up to 16 query
    heads per key head) and, when the step's chunk sizes are known on the host, chunks of MFMA_MIN_ROWS rows and more.
    Other chunks of GEMM_MIN_ROWS rows and more run as library GEMMs around a masked softmax kernel."""
    T = q.shape[0]
    if T == 0:
        return out
    if H % G:
        raise ValueError("masked_attention: heads must be a multiple of kv heads")
    Gv = G if v_heads is None else int(v_heads)
    if Gv < 1 or G % Gv:
        raise ValueError("masked_attention: the key heads are a multiple of the value heads")
    sink_v = sink if isinstance(sink, torch.Tensor) else None
    sink = sink_v is not None or bool(sink)
    if sink_v is not None and (sink_v.dtype != torch.float32 or sink_v.numel() != H or not sink_v.is_contiguous()):
        raise TypeError("masked_attention: one fp32 sink per query head")
    if bias is not None and (bias.dtype != torch.float32 or bias.dim() != 2 or bias.shape[0] != H
                             or not bias.is_contiguous()):
        raise TypeError("masked_attention: the distance bias is a contiguous fp32 [H, distances] table")
    if gate is not None and (gate.dtype != torch.float32 or gate.shape != (T, H) or gate.stride(1) != 1):
        raise TypeError("masked_attention: the gate is fp32 [T, H]")
    nd = rag.n_dec
    if not q.is_cuda:
        if nd:
            lens = rag.dec_lens.tolist()
            for i in range(nd):
                _attn_ref(q[i:i + 1], kc, vc, rag.dec_bt[i], lens[i], lens[i] - 1, H, G, dk, dv, scale, chunk, window,
                          sink, out[i:i + 1], out_scale, sink_v, bias, gate[i:i + 1] if gate is not None else None, Gv)
        if rag.n_pf:
            cu, ctx = rag.pf_cu.tolist(), rag.pf_ctx.tolist()
            for k in range(rag.n_pf):
                n = cu[k + 1] - cu[k]
                if n:
                    r0 = nd + cu[k]
                    _attn_ref(q[r0:r0 + n], kc, vc, rag.pf_bt[k], ctx[k], ctx[k] - n, H, G, dk, dv, scale, chunk,
                              window, sink, out[r0:r0 + n], out_scale, sink_v, bias,
                              gate[r0:r0 + n] if gate is not None else None, Gv)
        return out
    if q.dtype != kc.dtype or kc.dtype != vc.dtype or q.stride(1) != 1 or out.stride(1) != 1:
        raise TypeError("masked_attention: queries and pools share one dtype, rows are contiguous")
    bs = kc.shape[1]
    st = N.stream_ptr()
    common = (H, G, dk, dv, float(scale), int(chunk), int(window), int(sink), float(out_scale))
    nb = bias.shape[1] if bias is not None else 0
    ldg = gate.stride(0) if gate is not None else 0
    extra = (N.ptr(sink_v), N.ptr(bias), nb)  # the gate pointer moves with the rows a launch serves
    mfma_ok = q.dtype == torch.bfloat16 and q.stride(0) % 8 == 0 and MFMA_MIN_ROWS > 0 and \
        bool(N.hybrid_kernels().mxh_attention_mfma_ok(dk, dv))
    if nd:
        vis = rag.dec_max_len
        vis = min(vis, chunk) if chunk else min(vis, window) if window else vis
        dec_mfma = mfma_ok and H // G <= 16  # a wave's 16 rows are the query heads of one key / value head
        parts, plen = 1, 0
        if workspace is not None:
            plen = decode_part_len(nd, G * 4 if dec_mfma else H, vis)
            parts = -(-vis // plen)
            room = min(64, workspace[0].shape[0] // (nd * H))  # the merge holds one partition per lane
            if parts > room:
                parts = max(1, room)
                plen = -(-(-(-vis // parts)) // 64) * 64
        ml, po = (workspace[0], workspace[1]) if parts > 1 else (None, None)
        if dec_mfma:
            N.kcall("mxh_attention_decode_mfma", q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(), bs,
                    rag.dec_bt.data_ptr(), rag.dec_bt.stride(0), rag.dec_lens.data_ptr(), nd, out.data_ptr(),
                    out.stride(0), _is16(out), H, G, dk, dv, float(scale), int(chunk), int(window), int(sink),
                    float(out_scale), parts, plen if parts > 1 else 0, N.ptr(ml), N.ptr(po), *extra, N.ptr(gate), ldg,
                    Gv, int(p32), st)
        else:
            N.kcall("mxh_attention", q.data_ptr(), q.stride(0), _is16(q), kc.data_ptr(), vc.data_ptr(), bs,
                    rag.dec_bt.data_ptr(), rag.dec_bt.stride(0), None, rag.dec_lens.data_ptr(), nd, nd, 0,
                    out.data_ptr(), out.stride(0), _is16(out), *common, 0, parts, plen if parts > 1 else 0, N.ptr(ml),
                    N.ptr(po), *extra, N.ptr(gate), ldg, Gv, st)
    if rag.n_pf:
        lens = rag.pf_q_host if len(rag.pf_q_host) == rag.n_pf and len(rag.pf_ctx_host) == rag.n_pf else None

        def rows_kernel(row_off, n_rows):
            N.kcall("mxh_attention", q.data_ptr(), q.stride(0), _is16(q), kc.data_ptr(), vc.data_ptr(), bs,
                    rag.pf_bt.data_ptr(), rag.pf_bt.stride(0), rag.pf_cu.data_ptr(), rag.pf_ctx.data_ptr(), rag.n_pf,
                    n_rows, nd, out.data_ptr(), out.stride(0), _is16(out), *common, row_off, 1, 0, None, None, *extra,
                    N.ptr(gate), ldg, Gv, st)
        mfma = mfma_ok
        big = MFMA_MIN_ROWS if mfma else GEMM_MIN_ROWS
        if lens is None or max(lens) < big or (not mfma and 0 < chunk < GEMM_MIN_ROWS):
            rows_kernel(0, T - nd)  # (mask chunks shorter than a block of rows: few visible keys, the row kernel's case)
            return out
        r, run0 = 0, None  # run0: first row of a run of consecutive short chunks
        for k, n in enumerate(lens):
            if n >= big:
                if run0 is not None:
                    rows_kernel(run0, r - run0)
                    run0 = None
                qk, ok = q[nd + r:nd + r + n], out[nd + r:nd + r + n]
                gk = gate[nd + r:nd + r + n] if gate is not None else None
                if mfma:
                    N.kcall("mxh_attention_mfma", qk.data_ptr(), qk.stride(0), kc.data_ptr(), vc.data_ptr(), bs,
                            rag.pf_bt[k].data_ptr(), rag.pf_ctx_host[k] - n, n, ok.data_ptr(), ok.stride(0), _is16(out),
                            H, G, dk, dv, float(scale), int(chunk), int(window), int(sink), float(out_scale), *extra,
                            N.ptr(gk), ldg, Gv, int(p32), st)
                else:
                    _attn_gemm_chunk(qk, kc, vc, rag.pf_bt[k], rag.pf_ctx_host[k] - n, n, H, G, dk, dv, scale, chunk,
                                     window, sink, ok, out_scale, sink_v, bias, gk, Gv, p32)
            elif n and run0 is None:
                run0 = r
            r += n
        if run0 is not None:
            rows_kernel(run0, r - run0)
    return out


# ------------------------------------------------------------------------------------------------ convolution
def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, tails: torch.Tensor, rag: Ragged,
                out: torch.Tensor, silu: bool = True):
    """out_t = act(bias + sum_j w[:, j] * x_(t - taps + 1 + j)) per channel over each sequence's rows; the
    sequence's previous taps-1 inputs are read from (and its newest written back to) `tails` [slots, taps-1, C]
    fp32; a chunk that starts at position 0 reads zeros. x fp32 [T, C] (may be a column slice), w fp32 [C, taps],
    out fp32 [T, C]. A state slot < 0 (padding rows) reads zeros and stores nothing."""
    T, C = x.shape
    taps = w.shape[1]
    if T == 0:
        return out
    if not x.is_cuda:
        st, pos = rag.state.tolist(), rag.positions.tolist()
        for r0, n, si in rag.host_segments():
            slot = st[si]
            fresh = pos[r0] == 0 or slot < 0 or taps == 1
            prev = torch.zeros(taps - 1, C) if fresh else tails[slot].clone()
            full = torch.cat([prev, x[r0:r0 + n].float()], 0)
            y = torch.zeros(n, C)
            for j in range(taps):
                y += w[:, j] * full[j:j + n]
            if bias is not None:
                y += bias
            out[r0:r0 + n] = F.silu(y) if silu else y
            if slot >= 0 and taps > 1:
                tails[slot] = full[full.shape[0] - (taps - 1):]
        return out
    if taps > 16:
        raise ValueError("causal_conv: at most 16 taps")
    _f32c(x, "causal_conv")
    _f32c(out, "causal_conv")
    if tails.shape[1] != max(1, taps - 1) or tails.shape[2] != C or not tails.is_contiguous():
        raise ValueError("causal_conv: tails are [slots, taps - 1, channels]")
    N.kcall("mxh_causal_conv", x.data_ptr(), x.stride(0), w.data_ptr(), N.ptr(bias), taps, int(silu),
            tails.data_ptr(), rag.state.data_ptr(), rag.positions.data_ptr(), rag.n_dec, N.ptr(rag.pf_cu), rag.n_pf,
            out.data_ptr(), out.stride(0), T, C, N.stream_ptr())
    return out


# ------------------------------------------------------------------------------------------------ recurrences
def unit_norm_heads(x: torch.Tensor, heads: int, dim: int, eps: float, scale: float = 1.0, split: int | None = None,
                    scale2: float = 1.0):
    """In place on fp32 x [T, heads*dim]: every head becomes x / sqrt(sum(x^2) + eps) * scale; heads from index
    `split` on are multiplied by scale2 instead (queries and keys that lie side by side in one launch)."""
    T = x.shape[0]
    if T == 0:
        return x
    split = heads if split is None else split
    if not x.is_cuda:
        v = x.reshape(T, heads, dim)
        sc = torch.full((heads, 1), float(scale))
        sc[split:] = scale2
        x.copy_((v * torch.rsqrt(v.pow(2).sum(-1, keepdim=True) + eps) * sc).reshape(T, heads * dim))
        return x
    _f32c(x, "unit_norm_heads")
    N.kcall("mxh_unit_norm", x.data_ptr(), x.stride(0), heads, dim, float(eps), float(scale), int(split), float(scale2),
            T, N.stream_ptr())
    return x


def scan_coefs(a: torch.Tensor, b: torch.Tensor | None, A_log: torch.Tensor, dt_bias: torch.Tensor,
               decay: torch.Tensor, coef: torch.Tensor):
    """Per token and head: s = softplus(a + dt_bias), decay = exp(-exp(A_log) * s), coef = sigmoid(b) when b is
    given, else s. a, b fp32 [T, H] column slices; decay, coef fp32 [T, H] contiguous."""
    T, H = a.shape
    if T == 0:
        return
    if not a.is_cuda:
        s = F.softplus(a.float() + dt_bias, threshold=30.0)
        decay.copy_(torch.exp(-torch.exp(A_log) * s))
        coef.copy_(torch.sigmoid(b.float()) if b is not None else s)
        return
    N.kcall("mxh_scan_coefs", a.data_ptr(), a.stride(0), N.ptr(b), b.stride(0) if b is not None else 0,
            A_log.data_ptr(), dt_bias.data_ptr(), decay.data_ptr(), coef.data_ptr(), T, H, N.stream_ptr())


def channel_decay(z: torch.Tensor, bias: torch.Tensor | None, tau: float, out: torch.Tensor,
                  proj: torch.Tensor | None = None, rate_log: torch.Tensor | None = None):
    """out = sigmoid(x)^(1 / tau), computed as exp(log_sigmoid(x) / tau): the per-channel decay of gated linear
    attention; or, with `rate_log` (fp32 [heads], C / heads channels per head, tau unused),
    out = exp(-exp(rate_log[head]) * softplus(x)): a step size per channel under a learned rate per head. x = z + bias
    with z fp32 [T, C]; or, with `proj` (fp32 [R, C], contiguous), x = z proj + bias with z fp32 [T, R]: the second half of a low-rank projection, done in fp32 inside the same kernel. z may be a column
    slice; bias fp32 [C]; out fp32 [T, C] contiguous."""
    T, C = out.shape
    if T == 0:
        return out
    if z.shape != ((T, proj.shape[0]) if proj is not None else (T, C)) or (proj is not None and proj.shape[1] != C):
        raise ValueError("channel_decay: z is [T, C], or [T, R] beside a projection [R, C]")
    if not z.is_cuda:
        x = z.float() @ proj.float() if proj is not None else z.float()
        if bias is not None:
            x = x + bias.float()
        if rate_log is not None:
            rate = torch.exp(rate_log.float()).repeat_interleave(C // rate_log.numel())
            out.copy_(torch.exp(-rate * F.softplus(x, threshold=30.0)))
        else:
            out.copy_(torch.exp(F.logsigmoid(x) / tau))
        return out
    _f32c(z, "channel_decay")
    if rate_log is not None and (rate_log.dtype != torch.float32 or C % rate_log.numel()):
        raise ValueError("channel_decay: one fp32 rate per head, whole heads of channels")
    if not out.is_contiguous() or out.dtype != torch.float32 or tau <= 0:
        raise ValueError("channel_decay: contiguous fp32 output, tau > 0")
    if proj is not None and (proj.dtype != torch.float32 or not proj.is_contiguous()):
        raise TypeError("channel_decay: the projection is a contiguous fp32 [R, C] matrix")
    N.kcall("mxh_channel_decay", z.data_ptr(), z.stride(0), N.ptr(bias), float(1.0 / tau), out.data_ptr(), T, C,
            N.ptr(proj), proj.shape[0] if proj is not None else 0, N.ptr(rate_log),
            C // rate_log.numel() if rate_log is not None else 0, N.stream_ptr())
    return out


def state_scan(k: torch.Tensor, q: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, coef: torch.Tensor | None,
               skip: torch.Tensor | None, state: torch.Tensor, rag: Ragged, out: torch.Tensor, H: int, G: int, Nk: int,
               P: int, delta: bool, channel: bool = False, q_scale: float = 1.0, coef_sigmoid: bool = False):
    """Linear recurrence per sequence and head over the step's rows, in order:
        S <- decay_t S;  u = coef_t (v_t - S^T k_t) if delta else coef_t v_t;  S <- S + k_t u^T;
        o_t = S^T (q_scale q_t) (+ skip_h v_t)
    k, q fp32 [T, G*Nk] (head h reads group h // (H / G)), v fp32 [T, H*P], decay / coef fp32 [T, H], out fp32
    [T, H*P]; all may be column slices. With `channel` the decay is fp32 [T, H*Nk], one number per head and key
    channel (row n of S is multiplied by decay[h, n]: gated linear attention, or with `delta` a delta rule with a decay
    per key channel). A decay of shape [H] is one constant per head for every token (retention). coef = None means 1;
    with `coef_sigmoid` coef holds pre-activations (a column slice of a projection's output) and the write strength is
    their sigmoid.
    state fp32 [slots, H, P, Nk] (a column's Nk numbers are contiguous) is read at
    the sequence's slot unless its first row is at position 0 (then S starts at zero) and written back after its last
    row."""
    T = k.shape[0]
    if T == 0:
        return out
    if not k.is_cuda:
        st, pos = rag.state.tolist(), rag.positions.tolist()
        rep = H // G
        for r0, n, si in rag.host_segments():
            slot = st[si]
            S = torch.zeros(H, Nk, P) if (pos[r0] == 0 or slot < 0) else state[slot].transpose(1, 2).clone()
            for t in range(r0, r0 + n):
                kt = k[t].float().reshape(G, Nk).repeat_interleave(rep, 0)
                qt = q[t].float().reshape(G, Nk).repeat_interleave(rep, 0) * q_scale
                vt = v[t].float().reshape(H, P)
                dt = decay if decay.dim() == 1 else decay[t]
                S = S * (dt.reshape(H, Nk)[:, :, None] if channel else dt[:, None, None])
                cf = 1.0
                if coef is not None:
                    cf = (torch.sigmoid(coef[t].float()) if coef_sigmoid else coef[t])[:, None]
                u = cf * ((vt - torch.einsum("hnp,hn->hp", S, kt)) if delta else vt)
                S = S + kt[:, :, None] * u[:, None, :]
                o = torch.einsum("hnp,hn->hp", S, qt)
                if skip is not None:
                    o = o + skip[:, None] * vt
                out[t] = o.reshape(H * P)
            if slot >= 0:
                state[slot] = S.transpose(1, 2)
        return out
    for t_ in (k, q, v, out):
        _f32c(t_, "state_scan")
    if tuple(state.shape[1:]) != (H, P, Nk) or not state.is_contiguous() or not decay.is_contiguous() \
            or (coef is not None and (coef.stride(1) != 1 or coef.dtype != torch.float32)) or H % G or Nk > 256:
        raise ValueError("state_scan: state is [slots, H, P, N] with N <= 256, decay contiguous, coef fp32 [T, H]")
    if decay.shape[-1] != (H * Nk if channel else H) or (decay.dim() == 1 and channel) or decay.dtype != torch.float32:
        raise ValueError("state_scan: one fp32 decay per head, or per head and key channel")
    N.kcall("mxh_state_scan", k.data_ptr(), k.stride(0), q.data_ptr(), q.stride(0), v.data_ptr(), v.stride(0),
            decay.data_ptr(), 0 if decay.dim() == 1 else 1, N.ptr(coef),
            coef.stride(0) if coef is not None else 0, int(coef_sigmoid), N.ptr(skip), state.data_ptr(),
            rag.state.data_ptr(),
            rag.positions.data_ptr(), rag.n_dec, N.ptr(rag.pf_cu), rag.n_pf, out.data_ptr(), out.stride(0), H, G, Nk,
            P, int(delta), int(channel), float(q_scale), N.stream_ptr())
    return out


def gated_group_norm(y: torch.Tensor, gate: torch.Tensor, w: torch.Tensor | None, eps: float, group: int,
                     out: torch.Tensor, gate_first: bool, out_scale: float = 1.0, act: str = "silu",
                     proj: torch.Tensor | None = None):
    """Rows y [T, C] fp32 in groups of `group` columns, gate [T, C] fp32 (pre-activation), w fp32 whose length divides
    C (column c uses w[c % len(w)]; None: no weight). gate_first: z = y * act(gate), out = unit_rms_group(z) * w;
    otherwise out = unit_rms_group(y) * w * act(gate); act is "silu" or "sigmoid". With `proj` (fp32 [R, C], contiguous)
    the gate is [T, R] and its pre-activation is gate proj, summed in fp32 inside the kernel (the second half of a
    low-rank gate). out (fp32 or bf16, may be a column slice) gets out_scale times that."""
    T, C = y.shape
    if T == 0:
        return out
    if act not in ("silu", "sigmoid"):
        raise ValueError("gated_group_norm: the gate is a silu or a sigmoid")
    if w is None:
        w = _ones(y.device)
    if C % group or C % w.numel():
        raise ValueError("gated_group_norm: group size and weight length divide the row")
    if gate.shape != ((T, proj.shape[0]) if proj is not None else (T, C)) or (proj is not None and proj.shape[1] != C):
        raise ValueError("gated_group_norm: the gate is [T, C], or [T, R] beside a projection [R, C]")
    if not y.is_cuda:
        gp = gate.float() @ proj.float() if proj is not None else gate.float()
        g = F.silu(gp) if act == "silu" else torch.sigmoid(gp)
        z = (y.float() * g if gate_first else y.float()).reshape(T, C // group, group)
        z = (z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, C) * w.float().repeat(C // w.numel())
        out.copy_(((z if gate_first else z * g) * out_scale).to(out.dtype))
        return out
    _f32c(y, "gated_group_norm")
    _f32c(gate, "gated_group_norm")
    if proj is not None and (proj.dtype != torch.float32 or not proj.is_contiguous()):
        raise TypeError("gated_group_norm: the projection is a contiguous fp32 [R, C] matrix")
    N.kcall("mxh_gated_group_norm", y.data_ptr(), y.stride(0), gate.data_ptr(), gate.stride(0), w.data_ptr(),
            w.numel(), float(eps), group, int(gate_first), float(out_scale), out.data_ptr(), out.stride(0), _is16(out),
            T, C, int(act == "sigmoid"), N.ptr(proj), proj.shape[0] if proj is not None else 0, N.stream_ptr())
    return out


_ONES: dict = {}


def _ones(device) -> torch.Tensor:
    """A one-element fp32 tensor holding 1 (the weight of a norm without weights)."""
    t = _ONES.get(device)
    if t is None:
        t = _ONES[device] = torch.ones(1, dtype=torch.float32, device=device)
    return t


def diff_group_norm(a: torch.Tensor, b: torch.Tensor, lam: float, eps: float, group: int, out: torch.Tensor,
                    out_scale: float = 1.0):
    """out = unit_rms_group(a - lam * b) * out_scale over groups of `group` columns: two attention maps over the same
    values combined per head (differential attention) and normed without a weight. a, b fp32 [T, C] (column slices
    allowed), out fp32 or bf16 [T, C] (may be a column slice)."""
    T, C = a.shape
    if T == 0:
        return out
    if C % group or b.shape != a.shape:
        raise ValueError("diff_group_norm: two [T, C] inputs, whole groups")
    if not a.is_cuda:
        z = (a.float() - lam * b.float()).reshape(T, C // group, group)
        z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * out_scale
        out.copy_(z.reshape(T, C).to(out.dtype))
        return out
    _f32c(a, "diff_group_norm")
    _f32c(b, "diff_group_norm")
    if group > 8192:
        raise ValueError("diff_group_norm: groups of up to 8192 numbers")
    N.kcall("mxh_diff_group_norm", a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), float(lam), float(eps), group,
            float(out_scale), out.data_ptr(), out.stride(0), _is16(out), T, C, N.stream_ptr())
    return out


# ------------------------------------------------------------------------------------------------ feed-forward
GLU_ACTS = {"silu": 0, "gelu_tanh": 1, "relu2": 2}


def glu(a: torch.Tensor, b: torch.Tensor | None, bias_a: torch.Tensor | None, bias_b: torch.Tensor | None,
        out: torch.Tensor, scale: torch.Tensor | None = None, group: int = 0, scale_sigmoid: bool = False,
        act: str = "silu"):
    """out = act(a + bias_a) * (b + bias_b) [* factor] with act "silu" or "gelu_tanh" (0.5 z (1 + tanh(sqrt(2 / pi)
    (z + 0.044715 z^3)))); a, b fp32 [T, F] column slices, out fp32 or bf16 [T, F] (may be a column slice). `scale`
    fp32 [T, F / group] (column slice allowed) gives one factor per row and group of `group` columns, passed through a
    sigmoid first with `scale_sigmoid`. act "relu2" has no second operand (b = None) and the factor multiplies the
    INPUT: out = relu(factor * (a + bias_a))^2, an expert that is fed its routing weight times the token."""
    T, Fn = a.shape
    if T == 0 or Fn == 0:
        return out
    if act not in GLU_ACTS or (b is None) != (act == "relu2"):
        raise ValueError("glu: act is silu | gelu_tanh with two operands, or relu2 with one")
    if not a.is_cuda:
        x = a.float() + bias_a if bias_a is not None else a.float()
        s = None
        if scale is not None:
            s = torch.sigmoid(scale.float()) if scale_sigmoid else scale.float()
            s = s.repeat_interleave(group, 1)
        if act == "relu2":
            z = torch.relu(x * s if s is not None else x).pow(2)
        else:
            y = b.float() + bias_b if bias_b is not None else b.float()
            z = (F.silu(x) if act == "silu" else F.gelu(x, approximate="tanh")) * y
            if s is not None:
                z = z * s
        out.copy_(z.to(out.dtype))
        return out
    _f32c(a, "glu")
    if b is not None:
        _f32c(b, "glu")
    if scale is not None and (group <= 0 or Fn % group or scale.shape[1] != Fn // group):
        raise ValueError("glu: one factor per row and group of columns")
    N.kcall("mxh_glu", a.data_ptr(), a.stride(0), N.ptr(b), b.stride(0) if b is not None else 0, N.ptr(bias_a),
            N.ptr(bias_b), N.ptr(scale), scale.stride(0) if scale is not None else 0,
            group if scale is not None else Fn, int(scale_sigmoid), out.data_ptr(), out.stride(0), _is16(out), T, Fn,
            GLU_ACTS[act], N.stream_ptr())
    return out


def moe_route(logits: torch.Tensor, top: int, scale: float, weights: torch.Tensor, eps: float = 1e-20,
              bias: torch.Tensor | None = None, mode: str = "softmax"):
    """Router of a mixture of experts: s = softmax(logits + bias) over all E experts, the `top` largest are kept,
    divided by their sum (+ eps) and multiplied by `scale` (eps = 0, scale = 1: the softmax over the chosen logits
    alone). logits fp32 [T, E] (column slice allowed), bias fp32 [E]; weights fp32 [T, E] contiguous: the chosen
    experts' weights, 0 elsewhere. Ties go to the lower expert index. mode "sigmoid": the scores are
    sigmoid(logits + bias), the `top` largest are chosen and keep their scores as weights, times `scale`, not
    renormalised."""
    T, E = logits.shape
    if T == 0:
        return weights
    if not 0 < top <= E:
        raise ValueError("moe_route: 1 <= top <= experts")
    if mode not in ("softmax", "sigmoid"):
        raise ValueError("moe_route: softmax or sigmoid scores")
    if not logits.is_cuda:
        z = logits.float() + bias.float() if bias is not None else logits.float()
        weights.zero_()
        if mode == "sigmoid":
            tv, ti = torch.topk(z, top, dim=-1)
            weights.scatter_(1, ti, torch.sigmoid(tv) * scale)
            return weights
        tv, ti = torch.topk(torch.softmax(z, -1), top, dim=-1)
        weights.scatter_(1, ti, tv / (tv.sum(-1, keepdim=True) + eps) * scale)
        return weights
    _f32c(logits, "moe_route")
    if E > 1024:
        raise ValueError("moe_route: at most 1024 experts")
    N.kcall("mxh_moe_route", logits.data_ptr(), logits.stride(0), N.ptr(bias), T, E, top, float(scale), float(eps),
            weights.data_ptr(), int(mode == "sigmoid"), N.stream_ptr())
    return weights
