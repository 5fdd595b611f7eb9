"""Keronex (hyper-connection streams, a hashed pair embedding, differential attention over shared values, retention,
a delta rule with per-channel decays, dense and expert feed-forwards whose routing weight scales the expert's input) on
the engine against the plain float64 oracle of tests/oracle_keronex.py: every mechanism alone, whole prompts,
token-by-token decoding, prompt portions down to two tokens, unequal batches, reuse of freed blocks and state slots,
keys far back / at page borders / at the sequence's start with peaked softmax weights, odd sizes, long decoding, greedy
generation through the scheduler, graph replays, and the trace runner's command line.

Each engine test runs on the CPU plumbing path (fp32) and, marked gpu, on the HIP kernels in fp32 and bf16."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import oracle_keronex as O
from localai_tfp_amd.engine.engine import EngineConfig, LLMEngine
from localai_tfp_amd.models import keronex as KE
from localai_tfp_amd.ops import hybrid as HY
from localai_tfp_amd.ops.sampling import SamplingParams
from localai_tfp_amd.tokenizer import ByteTokenizer
from test_vugotar import _FB, close, engine, run_cuts, steps_of, toks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVS = ["cpu", GPU]
RUNS = [("cpu", "float32", 2e-4), pytest.param("cuda", "float32", 2e-4, marks=pytest.mark.gpu),
        pytest.param("cuda", "bfloat16", 6e-2, marks=pytest.mark.gpu)]
F64 = torch.float64

SHAPES = {
    # every mixer, a layer that runs another layer's tensors on a state of its own, both feed-forwards, three streams
    "plain": dict(hidden=64, vocab=97, pattern=("attention", "channel_delta", "retention", "retention"),
                  weights_of={3: 2}, heads=4, kv_heads=2, dim=16, vdim=16, r_heads=2, r_dim=16, r_vdim=16, d_heads=2,
                  d_kv_heads=1, d_dim=16, d_vdim=16, conv=4, rank_a=6, rank_g=5, mlps=("dense", "moe"), ff=96,
                  experts=4, top=2, expert_ff=32, shared_ff=32, streams=3, emb_scale=4.0, bigram=(61, 7, 3)),
    # sizes that differ from each other: dim != vdim, partial rotation and none, as many key heads as heads, two
    # taps, top == experts, no shared expert, a layer without a feed-forward, a large eps, one plain residual (no
    # stream tensors), no pair table, no embedding scale, a recurrent first layer, stacked projections of odd width
    "odd": dict(hidden=40, vocab=61, pattern=("retention", "attention", "channel_delta", "attention"),
                mlps=(None, "moe", "dense"), heads=3, kv_heads=3, dim=24, vdim=40, rot_dims=8, rot_base=300.0, scale=0.4,
                diff=0.2, r_heads=3, r_dim=20, r_vdim=12, r_rot_dims=0, d_heads=3, d_kv_heads=3, d_dim=20, d_vdim=12,
                conv=2, rank_a=3, rank_g=2, ff=50, experts=5, top=5, expert_ff=17, shared_ff=0, streams=None,
                bigram=None, eps=1e-3),
    # states wider than a lane keeps alone (160 and 96 numbers per column), value sizes that are no multiple of 64,
    # one expert of many, one key head for all heads, one tap (no carried inputs), ONE stream that still has its
    # tensors, hash multipliers far beyond the table
    "wide": dict(hidden=48, vocab=53, pattern=("attention", "channel_delta", "retention"), mlps=("moe", "dense", "moe"),
                 heads=4, kv_heads=1, dim=72, vdim=8, scale=0.2, diff=0.8, d_heads=2, d_kv_heads=2, d_dim=160,
                 d_vdim=80, conv=1, rank_a=16, rank_g=1, r_heads=2, r_dim=96, r_vdim=72, r_rot_dims=32, ff=64,
                 experts=9, top=1, expert_ff=16, shared_ff=24, streams=1, emb_scale=0.5, bigram=(7, 100003, 50021)),
    # nothing a multiple of eight: width, vocabulary, head sizes, expert widths, inner sizes; five streams, five taps
    "ragged": dict(hidden=44, vocab=101, pattern=("channel_delta", "attention", "retention"), heads=5, kv_heads=5,
                   dim=20, vdim=12, rot_dims=20, scale=0.3, diff=0.35, d_heads=6, d_kv_heads=2, d_dim=10, d_vdim=6,
                   conv=5, rank_a=5, rank_g=3, r_heads=3, r_dim=10, r_vdim=6, decay=(0.5, 0.97, 1.0), ff=30, experts=3,
                   top=2, expert_ff=10, shared_ff=6, streams=5, emb_scale=2.0, bigram=(13, 5, 11)),
}


def build(device="cpu", dtype="float32", seed=0, **kw):
    cfg = KE.make_config(**kw)
    get = KE.synthetic_source(cfg, seed)
    model = KE.KeronexModel.load(cfg, get, torch.device(device), getattr(torch, dtype))
    return cfg, {k: get(k) for k in get.names}, model


def oracle(cfg, tensors, tokens, layers=None):
    return O.forward(cfg.to_json(), tensors.get, tokens, layers).float()


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
def test_pair_embedding_carries_the_previous_token(dev):
    """Two sequences fed in portions (a chunk beside a decoded token, chunks of two) through slots that hold another
    sequence's last token: the row of the pair table follows the true previous token, position 0 takes the extra row."""
    g = torch.Generator().manual_seed(3)
    V, C, B, mp, mc, S = 50, 24, 11, 100003, 7, 3
    table, pair = torch.randn(V, C, generator=g), torch.randn(B + 1, C, generator=g)
    a, b = toks(9, V, 1), toks(6, V, 2)
    want = {}
    for key, t in (("a", a), ("b", b)):
        want[key] = table.double()[t] * 1.5 + pair.double()[O.pair_rows(t, B, mp, mc)]
    rows = O.pair_rows(a, B, mp, mc)
    assert rows[0] == B and rows != O.pair_rows(a, B, 1, 1)  # (the multipliers matter)
    last = torch.tensor([41, 17, 33], dtype=torch.int32, device=dev)  # stale tokens of earlier owners
    td, pd = table.to(dev), pair.to(dev)
    got = {"a": [], "b": []}
    # (decode rows first, then chunks) a: slot 2, b: slot 0
    steps = [([], [("a", 0, 4), ("b", 0, 2)]), ([("b", 2)], [("a", 4, 2)]), ([("a", 6), ("b", 3)], []),
             ([("a", 7)], [("b", 4, 2)]), ([("a", 8)], [])]
    seqs, slot = {"a": a, "b": b}, {"a": 2, "b": 0}
    for dec, chunks in steps:
        tk = [seqs[k][p] for k, p in dec] + [x for k, p, n in chunks for x in seqs[k][p:p + n]]
        pos = [p for _, p in dec] + [p + i for _, p, n in chunks for i in range(n)]
        fb = _FB(len(dec), [n for _, _, n in chunks], pos, [slot[k] for k, _ in dec] + [slot[k] for k, _, _ in chunks], dev)
        out = torch.full((len(tk), S * C), 9.0, device=dev)
        HY.embed_pair(td, pd, torch.tensor(tk, dtype=torch.int32, device=dev), HY.Ragged(fb), last, 1.5, mp, mc, B, out,
                      copies=S)
        assert torch.equal(out[:, :C], out[:, C:2 * C]) and torch.equal(out[:, :C], out[:, 2 * C:])
        r = 0
        for k, _ in dec:
            got[k].append(out[r:r + 1, :C].cpu())
            r += 1
        for k, _, n in chunks:
            got[k].append(out[r:r + n, :C].cpu())
            r += n
    for k in got:
        close(torch.cat(got[k]), want[k], 1e-6)
    assert last.tolist() == [b[-1], 17, a[-1]]
    out = torch.empty(3, C, device=dev)  # no pair table: the scaled embedding alone
    fb = _FB(0, [3], [0, 1, 2], [1], dev)
    HY.embed_pair(td, None, torch.tensor(a[:3], dtype=torch.int32, device=dev), HY.Ragged(fb), None, 0.25, 0, 0, 1, out)
    close(out, table.double()[a[:3]] * 0.25, 1e-6)


@pytest.mark.parametrize("dev", DEVS)
def test_stream_update_read_and_sum(dev):
    g = torch.Generator().manual_seed(5)
    eps = 0.3  # a large eps shows whether it sits inside the root
    for S, C, M in ((1, 40, 3), (3, 72, 5), (4, 2100, 2), (7, 300, 2), (8, 64, 2), (2, 9000, 2), (3, 5000, 2), (11, 300, 3),
                    (32, 70, 2)):
        xs = torch.randn(M, S, C, generator=g) * 2
        y = torch.randn(M, C + 3, generator=g)
        mix, wo, wi = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
        w = 0.2 * torch.randn(C, generator=g)
        old = [xs[:, s].double() for s in range(S)]
        new = O.hyper_write(old, y[:, 3:].double(), mix.double(), wo.double())
        h = O.offset_norm(O.hyper_read(new, wi.double()), w, eps)
        xd = xs.reshape(M, S * C).clone().to(dev)
        h32, h16 = torch.empty(M, C, device=dev), torch.empty(M, C, device=dev, dtype=torch.bfloat16)
        tot = torch.empty(M, C, device=dev)
        HY.hyper_step(xd, y.to(dev)[:, 3:], mix.to(dev), wo.to(dev), wi.to(dev), w.to(dev), eps, h32, h16, tot)
        close(xd.view(M, S, C), torch.stack(new, 1), 1e-5)
        close(h32, h, 1e-5)
        close(h16.float(), h, 1e-2)
        close(tot, sum(new), 1e-5)
        # a read alone (the first sublayer), then an update alone with the sum (after the last one)
        xd = xs.reshape(M, S * C).clone().to(dev)
        HY.hyper_step(xd, None, None, None, wi.to(dev), w.to(dev), eps, h32)
        close(h32, O.offset_norm(O.hyper_read(old, wi.double()), w, eps), 1e-5)
        assert torch.equal(xd.cpu(), xs.reshape(M, S * C))
        HY.hyper_step(xd, y.to(dev)[:, 3:], mix.to(dev), wo.to(dev), None, None, eps, total=tot)
        close(tot, sum(new), 1e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_rotation_of_half_pairs_in_place(dev):
    g = torch.Generator().manual_seed(2)
    for heads, dim, rot, base in ((3, 16, 16, 10000.0), (2, 24, 8, 300.0), (4, 72, 40, 1e6), (2, 20, 0, 10.0)):
        T = 6
        pos = [0, 1, 2, 977, 978, 3000]
        x = torch.randn(T, heads * dim + 4, generator=g)
        want = torch.zeros(T, heads, dim, dtype=F64)
        for i, p in enumerate(pos):  # the oracle turns row t by position t: build a sequence that holds row i at p
            seq = torch.zeros(p + 1, heads, dim, dtype=F64)
            seq[p] = x[i, 4:].double().reshape(heads, dim)
            want[i] = O.rotate_halves(seq, rot, base)[p]
        want[:, 1:] *= 0.5  # heads from index 1 on take the second scale
        xd = x.clone().to(dev)
        HY.rope_rows(xd[:, 4:], torch.tensor(pos, dtype=torch.int32, device=dev), heads, dim, rot, base, half=True,
                     scale=1.0, split=1, scale2=0.5)
        close(xd[:, 4:].reshape(T, heads, dim), want, 5e-4)  # fp32 angles at position 3000
        assert torch.equal(xd[:, :4].cpu(), x[:, :4])


def _diff_attention_case(dev, dt, H, G, dk, dv, rot, n, cuts, bs, scale, lam, diff, plant=()):
    """Rotation + append of both maps' keys and one set of values, attention over twice the heads reading value head
    g % G, then the combination and the head norm, in portions through shuffled pages. `plant` = [(query position, key
    position, map)]: the query's map is made a large multiple of the key's, so that one score stands out."""
    g = torch.Generator().manual_seed(7)
    md = getattr(torch, dt)
    q = torch.randn(n, H, 2, dk, generator=g)
    k = torch.randn(n, G, 2, dk, generator=g)
    v = torch.randn(n, G, dv, generator=g)
    eps = 1e-6
    base = 500.0
    qr = O.rotate_halves(q.double().reshape(n, 2 * H, dk), rot, base).reshape(n, H, 2, dk)
    kr = O.rotate_halves(k.double().reshape(n, 2 * G, dk), rot, base).reshape(n, G, 2, dk)
    for qi, kj, mp in plant:  # planted after the rotation, and un-rotated below: the kernel's rotation must restore it
        for h in range(H):
            qr[qi, h, mp] = kr[kj, h // (H // G), mp] * 6.0
    if plant:
        def unrotate(x):  # the inverse rotation: by the negated angle = the rotation of the mirrored pair
            n2 = rot // 2
            y = x.clone()
            if rot:
                y[..., n2:rot] = -y[..., n2:rot]
                y = O.rotate_halves(y, rot, base)
                y[..., n2:rot] = -y[..., n2:rot]
            return y
        q = unrotate(qr.reshape(n, 2 * H, dk)).reshape(n, H, 2, dk).float()
        qr = O.rotate_halves(q.double().reshape(n, 2 * H, dk), rot, base).reshape(n, H, 2, dk)
    if md == torch.bfloat16:  # the pools and the query operand hold bf16: the oracle reads the same rounded numbers
        qr, kr, vv = qr.float().to(md).double(), kr.float().to(md).double(), v.to(md).double()
    else:
        vv = v.double()
    want = O.differential_attention(qr, kr, vv, scale, lam, diff, eps).reshape(n, H * dv)
    # the package's layout: maps first, then heads
    qm = q.transpose(1, 2).reshape(n, 2 * H * dk)
    km = k.transpose(1, 2).reshape(n, 2 * G * dk)
    nb = -(-n // bs)
    table = torch.randperm(nb + 3, generator=g)[:nb].tolist()  # pages out of order
    kc = torch.full((nb + 3, bs, 2 * G * dk), 7.0, dtype=md, device=dev)  # stale numbers in unused slots
    vc = torch.full((nb + 3, bs, G * dv), -5.0, dtype=md, device=dev)
    wide = torch.cat([torch.randn(n, 3, generator=g), qm, km, v.reshape(n, G * dv)], 1).to(dev)
    got = torch.empty(n, H * dv + 5, device=dev, dtype=md)
    part = (torch.empty(2 * H * 8, 2, device=dev), torch.empty(2 * H * 8, dv, device=dev))  # room for eight partitions
    for n_dec, chunks, at in steps_of(n, cuts):
        c = 1 if n_dec else chunks[0]
        rws = list(range(at, at + c))
        slots = [table[p // bs] * bs + p % bs for p in rws]
        fb = _FB(n_dec, chunks, rws, [0], dev, slots, dec_bt=[table] if n_dec else None,
                 dec_lens=[at + 1] if n_dec else None, pf_bt=None if n_dec else [table],
                 pf_ctx=None if n_dec else [at + c])
        qo = torch.empty(c, 2 * H * dk, device=dev, dtype=md)
        w = wide[at:at + c]
        c0, c1 = 3 + 2 * H * dk, 3 + 2 * (H + G) * dk
        HY.rope_norm_append(w[:, 3:c0], w[:, c0:c1], w[:, c1:], fb.positions, 2 * H, 2 * G, dk, dv, rot, base, False, eps,
                            qo, kc, vc, fb.slots, half=True, v_heads=G)
        att = torch.empty(c, 2 * H * dv, device=dev)
        HY.masked_attention(qo, kc, vc, HY.Ragged(fb), 2 * H, 2 * G, dk, dv, scale, att, workspace=part, v_heads=G,
                            p32=True)
        HY.diff_group_norm(att[:, :H * dv], att[:, H * dv:], lam, eps, dv, got[at:at + c, 5:], out_scale=1.0 - diff)
    return got[:, 5:].float(), want


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("gemm_rows", [64, 8])
def test_differential_attention_pages_far_keys_and_portions(dev, dt, tol, gemm_rows, monkeypatch):
    """Planted keys carry nearly all of one map's weight: far back behind 260 keys, across a page border, at the
    query's own position and at position 0, in prompt portions and in rows decoded alone (split into partitions); the
    long portions also through the library-GEMM route (and from 8 rows on, so that short ones take it too)."""
    monkeypatch.setattr(HY, "GEMM_MIN_ROWS", gemm_rows)
    monkeypatch.setattr(HY, "DECODE_WAVES", 16)  # decode rows split into partitions of 64 keys
    tol = 3e-2 if dt == "bfloat16" else 2e-4  # (outputs are unit-RMS heads of a difference: a few bf16 steps)
    plant = [(270, 3, 0), (271, 0, 1), (100, 95, 0), (101, 96, 1), (150, 150, 0), (268, 15, 1), (269, 16, 0), (5, 0, 0)]
    got, want = _diff_attention_case(dev, dt, 4, 2, 24, 40, 8, 272, [97, 2, 80, 3, 70, 16] + [1] * 4, 16, 0.5, 0.7, 0.3,
                                     plant)
    close(got, want, tol)
    # head sizes of the matrix-core kernels (exact weights keep them on the row kernel / GEMM route), one key head
    got, want = _diff_attention_case(dev, dt, 3, 1, 64, 128, 64, 150, [70, 64, 2] + [1] * 14, 16, 0.3, -0.4, 0.5,
                                     [(149, 1, 0), (140, 63, 1), (141, 64, 0)])
    close(got, want, tol)
    # whole rotation, dim == vdim, as many key heads as heads, a page of 4 tokens
    got, want = _diff_attention_case(dev, dt, 2, 2, 16, 16, 16, 40, [9, 1, 1, 20, 2, 7], 4, 1.0, 1.3, 0.1,
                                     [(39, 3, 1), (38, 4, 0), (20, 19, 1)])
    close(got, want, tol)


@pytest.mark.parametrize("dev", DEVS)
def test_second_map_cancels_the_first(dev):
    """Equal maps and lam = 1 leave nothing but rounding; lam = 0 is one softmax attention, normed."""
    got, want = _diff_attention_case(dev, "float32", 2, 1, 16, 24, 0, 30, [30], 16, 0.4, 0.0, 0.25)
    close(got, want, 2e-4)
    n, H, dv = 12, 2, 8
    a = torch.randn(n, H * dv, generator=torch.Generator().manual_seed(1))
    out = torch.empty(n, H * dv, device=dev)
    HY.diff_group_norm(a.to(dev), (a * 0.5).to(dev), 2.0, 1e-2, dv, out, 0.7)
    assert float(out.abs().max()) < 1e-5  # (a - 2 * a / 2) / sqrt(0 + eps)
    big = torch.randn(2, 2 * 5000, generator=torch.Generator().manual_seed(2))  # groups beyond the register budget
    out = torch.empty(2, 2 * 5000, device=dev)
    HY.diff_group_norm(big.to(dev), big.flip(1).contiguous().to(dev), 0.3, 1e-6, 5000, out, 0.9)
    z = (big.double() - 0.3 * big.flip(1).double()).reshape(2, 2, 5000)
    close(out.view(2, 2, 5000), O.unit_rms(z, 1e-6) * 0.9, 1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("H,G,N,P", [(2, 1, 16, 16), (3, 3, 20, 12), (2, 2, 160, 80), (6, 2, 10, 6), (2, 1, 64, 128)])
def test_recurrences_in_portions(dev, H, G, N, P):
    """Retention (a constant decay per head) and the delta rule with a decay per key channel and the sigmoid of the
    write strength applied while staging: portions of 1 to 40 tokens, a dirty slot taken over, against the oracle."""
    g = torch.Generator().manual_seed(11)
    n, cuts = 75, [3, 2, 19, 1, 1, 40, 2, 7]
    k = torch.nn.functional.normalize(torch.randn(n, G, N, generator=g), dim=-1)
    q = torch.randn(n, G, N, generator=g) * N ** -0.5
    v = torch.randn(n, H, P, generator=g)
    b = torch.randn(n, H + 2, generator=g) * 2
    dec = torch.sigmoid(torch.randn(n, H, N, generator=g) * 2 + 2)
    const = torch.tensor([1.0 - 2.0 ** (-2 - h) for h in range(H)])
    rep = H // G
    kd, qd = k.double().repeat_interleave(rep, 1), q.double().repeat_interleave(rep, 1)
    want_d = O.channel_delta_rule(qd, kd, v.double(), torch.sigmoid(b[:, 2:].double()), dec.double())
    want_r = O.retention(qd * 0.5, kd, v.double(), const.double())
    for kind, want in (("delta", want_d), ("retention", want_r)):
        state = torch.full((3, H, P, N), 3.0, device=dev)  # slot 1 held another sequence
        got = torch.empty(n, H * P + 1, device=dev)
        kk, qq, vv = (x.reshape(n, -1).to(dev) for x in (k, q, v))
        for n_dec, chunks, at in steps_of(n, cuts):
            c = 1 if n_dec else chunks[0]
            fb = _FB(n_dec, chunks, list(range(at, at + c)), [1], dev)
            sl = slice(at, at + c)
            if kind == "delta":
                HY.state_scan(kk[sl], qq[sl], vv[sl], dec.reshape(n, H * N).to(dev)[sl].contiguous(), b.to(dev)[sl, 2:],
                              None, state, HY.Ragged(fb), got[sl, 1:], H, G, N, P, delta=True, channel=True,
                              coef_sigmoid=True)
            else:
                HY.state_scan(kk[sl], qq[sl], vv[sl], const.to(dev), None, None, state, HY.Ragged(fb), got[sl, 1:], H, G,
                              N, P, delta=False, q_scale=0.5)
        close(got[:, 1:].reshape(n, H, P), want, 2e-5)
        assert float(state[0].min()) == 3.0 and float(state[2].max()) == 3.0


@pytest.mark.parametrize("dev", DEVS)
def test_decays_gates_activations_and_router(dev):
    g = torch.Generator().manual_seed(4)
    T, H, N, R = 5, 3, 20, 6
    z, bias = torch.randn(T, R + 2, generator=g), torch.randn(H * N, generator=g)
    proj, rate = torch.randn(R, H * N, generator=g), torch.randn(H, generator=g)
    x = z[:, 2:].double() @ proj.double() + bias.double()
    want = torch.exp(-torch.exp(rate.double()).repeat_interleave(N) * torch.log1p(torch.exp(x)))
    out = torch.empty(T, H * N, device=dev)
    HY.channel_decay(z.to(dev)[:, 2:], bias.to(dev), 1.0, out, proj=proj.to(dev), rate_log=rate.to(dev))
    close(out, want, 1e-5)
    # head norm with a shared weight, times the sigmoid of a low-rank gate; and without a weight, times silu
    P = 12
    y, gz = torch.randn(T, H * P, generator=g) * 3, torch.randn(T, R, generator=g)
    gp, w = torch.randn(R, H * P, generator=g), 1.0 + 0.2 * torch.randn(P, generator=g)
    eps = 0.05
    want = (O.unit_rms(y.double().reshape(T, H, P), eps) * w.double()).reshape(T, H * P)
    want = want * torch.sigmoid(gz.double() @ gp.double())
    for md, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        out = torch.empty(T, H * P, device=dev, dtype=md)
        HY.gated_group_norm(y.to(dev), gz.to(dev), w.to(dev), eps, P, out, gate_first=False, act="sigmoid",
                            proj=gp.to(dev))
        close(out.float(), want, tol)
    gs = torch.randn(T, H * P, generator=g)
    out = torch.empty(T, H * P, device=dev)
    HY.gated_group_norm(y.to(dev), gs.to(dev), None, eps, P, out, gate_first=False)
    want = O.unit_rms(y.double().reshape(T, H, P), eps).reshape(T, H * P) * gs.double() * torch.sigmoid(gs.double())
    close(out, want, 1e-5)
    # activations: the tanh form of gelu as a gated unit; the squared ReLU of a scaled input
    a, b = torch.randn(T, 33, generator=g) * 3, torch.randn(T, 33, generator=g)
    out = torch.empty(T, 33, device=dev)
    HY.glu(a.to(dev), b.to(dev), None, None, out, act="gelu_tanh")
    close(out, O.gelu_tanh(a.double()) * b.double(), 1e-5)
    E, Fe = 3, 11
    rw = torch.tensor([[0.0, 0.7, 0.2], [0.9, 0.0, 0.0], [0.3, 0.3, 0.3], [0.0, 0.0, 1.0], [0.5, 0.0, 0.25]])
    out = torch.empty(T, E * Fe, device=dev)
    HY.glu(a.to(dev), None, None, None, out, scale=rw.to(dev), group=Fe, act="relu2")
    close(out, torch.relu(a.double() * rw.double().repeat_interleave(Fe, 1)) ** 2, 1e-5)
    HY.glu(a.to(dev), None, None, None, out, act="relu2")
    close(out, torch.relu(a.double()) ** 2, 1e-5)
    # router: sigmoid scores, the largest keep theirs, nothing is renormalised
    for E, top in ((7, 1), (7, 3), (5, 5), (130, 4)):
        lg = torch.randn(T, E + 1, generator=g) * 2
        want = torch.zeros(T, E, dtype=F64)
        for t in range(T):
            for e, wgt in O.route(torch.sigmoid(lg[t, 1:].double()), top):
                want[t, e] = wgt
        out = torch.empty(T, E, device=dev)
        HY.moe_route(lg.to(dev)[:, 1:], top, 1.0, out, 0.0, mode="sigmoid")
        close(out, want, 1e-5)
        assert int((out > 0).sum()) == T * top


# ------------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_portions_and_decoding(dev, dt, tol, shape):
    cfg, tensors, model = build(dev, dt, seed=5, **SHAPES[shape])
    t = toks(75, cfg.vocab, 1)
    want = oracle(cfg, tensors, t)
    eng = engine(model, 80)
    b16 = dt == "bfloat16"
    if b16 and shape in ("odd", "ragged"):  # some 40 numbers wide: single rows carry several times the typical rounding
        tol *= 2
    close(run_cuts(eng, "whole", t, [75]), want, tol, b16)
    close(run_cuts(eng, "decode", t, [40] + [1] * 35), want, tol, b16)
    close(run_cuts(eng, "cuts", t, [3, 2, 19, 2, 1, 1, 30, 2, 7, 1, 1, 1, 5]), want, tol, b16)
    close(run_cuts(eng, "first", t[:9], [1] * 9), want[:9], tol, b16)  # the first tokens, one by one from position 0
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 4


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("kind", ["retention", "channel_delta", "attention"])
def test_models_of_one_kind_of_layer(dev, dt, tol, kind):
    """Recurrent layers only (the paged pool is empty, blocks are bookkeeping) and attention layers only (the state
    slots hold the previous token alone), the last two layers on the first one's tensors."""
    kw = dict(SHAPES["plain"], pattern=(kind,) * 3, weights_of={1: 0, 2: 0}, mlps=("moe",))
    cfg, tensors, model = build(dev, dt, seed=13, **kw)
    assert (model.cache_ranks() == []) == (kind != "attention") and len(model.weights) == 1
    t = toks(60, cfg.vocab, 3)
    want = oracle(cfg, tensors, t)
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=64, max_model_len=64, block_size=16, use_graphs=False,
                      overlap=False, native_scheduler=False, logits_rows=64, gemm_autotune=False,
                      num_blocks=9 if kind == "attention" else 0)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
    b16 = dt == "bfloat16"
    close(run_cuts(eng, "a", t, [60]), want, tol, b16)
    close(run_cuts(eng, "b", t, [7, 2, 30] + [1] * 21), want, tol, b16)


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_residual_after_every_layer(dev, dt, tol):
    cfg, tensors, model = build(dev, dt, seed=9, **SHAPES["plain"])
    t = toks(30, cfg.vocab, 2)
    layers = []
    oracle(cfg, tensors, t, layers)
    eng = engine(model, 32)
    for r in range(1, len(layers) + 1):
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
    portions of some beside single tokens of others; finished requests hand their blocks and slot (recurrent states,
    convolution inputs, previous token) to new ones. Every request's logits equal those it gets alone."""
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
        close(torch.cat(got[k]), want[k], tol, dt == "bfloat16")
        # and the same request alone, in the same number format: no router tie falls differently here
        alone = run_cuts(eng, "alone-" + k, reqs[k], [len(reqs[k])])
        close(torch.cat(got[k]), alone, 2e-4 if dt == "float32" else 4e-3)
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 3


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_peaked_attention_far_keys_and_long_decode(dev, dt, tol):
    """A large score scale makes single keys dominate both maps, so a lost or shifted key anywhere in a long prompt
    (page borders, position 0) moves the logits; then 70 tokens decoded one by one while the decayed states are
    carried on."""
    kw = dict(SHAPES["plain"], scale=2.5, rot_base=50.0)
    cfg, tensors, model = build(dev, dt, seed=21, **kw)
    t = toks(260, cfg.vocab, 8)
    want = oracle(cfg, tensors, t)
    eng = engine(model, max_tokens=272, seqs=2)
    got = run_cuts(eng, "x", t, [187, 3] + [1] * 70)
    close(got, want, tol * 2, rms=dt == "bfloat16")


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("dim,vdim,heads,kv", [(64, 128, 8, 2), (128, 64, 3, 1)])
def test_matrix_core_head_sizes_through_the_engine(dev, dt, tol, dim, vdim, heads, kv):
    """Head sizes of 64 / 128: a prompt in portions that end inside 16-row tiles, decoded rows behind enough keys to be
    split into partitions, recurrent heads of 64 and 128 numbers."""
    kw = dict(hidden=128, vocab=211, pattern=("attention", "channel_delta", "retention"), heads=heads, kv_heads=kv,
              dim=dim, vdim=vdim, scale=1.5 * dim ** -0.5, d_heads=2, d_kv_heads=1, d_dim=128, d_vdim=64, r_heads=2,
              r_dim=64, r_vdim=128, rank_a=4, rank_g=4, mlps=("moe", "dense"), ff=128, experts=4, top=2, expert_ff=64,
              shared_ff=64, streams=2, bigram=(251, 31, 17))
    cfg, tensors, model = build(dev, dt, seed=17, **kw)
    t = toks(330, cfg.vocab, 9)
    want = oracle(cfg, tensors, t)
    eng = engine(model, max_tokens=336, seqs=2)
    b16 = dt == "bfloat16"
    close(run_cuts(eng, "x", t, [203, 17, 2, 41, 1, 1, 1, 33] + [1] * 31), want, tol, b16)
    close(run_cuts(eng, "y", t[:100], [100]), want[:100], tol, b16)


def _random_shape(rng):
    nl = rng.randint(2, 6)
    pattern, weights_of, seen = [], {}, {}
    for i in range(nl):
        kind = rng.choice(["attention", "retention", "channel_delta"])
        pattern.append(kind)
        if kind in seen and rng.random() < 0.3:
            weights_of[i] = seen[kind]
        else:
            seen.setdefault(kind, i)
    nm = rng.randint(1, 3)
    mlps = tuple(rng.choice(["moe", "dense", None]) for _ in range(nm))
    # a layer that runs another's tensors has that layer's feed-forward too: make_config copies the whole entry
    kv, dkv, experts = rng.choice([1, 2, 3]), rng.choice([1, 2]), rng.choice([2, 3, 4, 8, 16])
    dim, ddim, rdim = rng.choice([16, 32, 48, 64]), rng.choice([16, 32, 64, 128]), rng.choice([16, 32, 96])
    rh = rng.choice([1, 2, 4])
    return dict(hidden=rng.choice([64, 96, 160]), vocab=rng.choice([97, 256, 1000]), pattern=tuple(pattern),
                weights_of=weights_of, heads=kv * rng.choice([1, 2, 3]), kv_heads=kv, dim=dim,
                vdim=rng.choice([16, 32, 64, 128]), scale=rng.choice([0.05, 0.1, 0.2]), diff=rng.choice([0.1, 0.5, 0.8]),
                rot_dims=rng.choice([0, 8, dim]), rot_base=rng.choice([100.0, 1e4, 1e6]), r_heads=rh, r_dim=rdim,
                r_vdim=rng.choice([16, 32, 96]), r_rot_dims=rng.choice([0, 16, rdim]),
                decay=[rng.choice([0.9, 0.99, 0.999, 1.0]) for _ in range(rh)], d_heads=dkv * rng.choice([1, 2]),
                d_kv_heads=dkv, d_dim=ddim, d_vdim=rng.choice([16, 32, 96]), conv=rng.choice([1, 2, 4]),
                rank_a=rng.choice([1, 4, 16]), rank_g=rng.choice([1, 4, 16]), mlps=mlps, ff=rng.choice([48, 128]),
                experts=experts, top=rng.randint(1, experts), expert_ff=rng.choice([16, 40]),
                shared_ff=rng.choice([0, 32, 96]), streams=rng.choice([None, 1, 2, 4, 6]),
                emb_scale=rng.choice([1.0, 8.0]), bigram=rng.choice([None, (31, 5, 3), (499, 113, 19)]),
                eps=rng.choice([1e-6, 1e-5]))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_configurations_and_schedules(dev, seed):
    """Drawn sizes, layer orders and shared tensors; five requests fed through four live slots in drawn portions
    (single tokens beside portions of up to 150, requests left out of steps, blocks and slots handed on) in a pool that
    holds the four largest but not all five. fp32 only: every position agrees with the oracle."""
    import random
    rng = random.Random(seed)
    cfg, tensors, model = build(dev, "float32", seed=seed, **_random_shape(rng))
    g = torch.Generator().manual_seed(seed)
    reqs = {"r%d" % i: torch.randint(0, cfg.vocab, (n,), generator=g).tolist()
            for i, n in enumerate(rng.sample([5, 40, 90, 150, 230], 5))}
    want = {k: oracle(cfg, tensors, v) for k, v in reqs.items()}
    eng = engine(model, max_tokens=1024, seqs=4, blocks=34 + 1)  # 16-token pages: 1 + 3 + 6 + 10 + 15 would be 35
    pending, live, at, got = list(reqs), [], {}, {k: [] for k in reqs}
    while pending or live:
        while pending and len(live) < 4 and (not live or rng.random() < 0.5):
            live.append(pending.pop(0))
            at[live[-1]] = 0
        entries, end = [], []
        for k in list(live):
            if rng.random() < 0.15 and len(live) > 1:
                continue  # left out of this step
            n = min(len(reqs[k]) - at[k], rng.choice([1, 1, 1, 2, 3, 16, 37, 64, 150]))
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                live.remove(k)
                end.append(k)
        if not entries:
            continue
        out = eng.replay_step(entries, end)
        r = 0
        for k, tk, _ in entries:
            got[k].append(out[r:r + len(tk)])
            r += len(tk)
    for k in reqs:
        close(torch.cat(got[k]), want[k], 2e-4)
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 4


# ------------------------------------------------------------------------------------------------ serving path
@pytest.mark.parametrize("dev,dt", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("native", [False, True])
def test_greedy_generation_through_the_scheduler(dev, dt, native):
    """engine.submit: chunked prefill, continuous batching of three requests, greedy sampling; each request's tokens
    equal the oracle's greedy continuation (the pair embedding reads every sampled token as the next one's previous)."""
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
    cfg, tensors, model = build("cuda", "float32", seed=4, **SHAPES["ragged"])
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


def test_preempted_request_recomputes_its_state():
    """A pool too small for both requests' growth: one is preempted, loses its blocks and state slot, and is
    recomputed from position 0 later; both still produce the oracle's greedy tokens."""
    cfg, tensors, model = build("cpu", "float32", seed=8, **SHAPES["plain"])
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=64, max_model_len=128, block_size=16, num_blocks=8,
                      use_graphs=False, native_scheduler=False, gemm_autotune=False)
    eng = LLMEngine(model, ByteTokenizer(cfg.vocab), ec)
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
    cfg = KE.make_config(**SHAPES["odd"])
    get = KE.synthetic_source(cfg, 1)
    KE.save_checkpoint(cfg, get, str(tmp_path))
    assert KE.is_keronex_dir(str(tmp_path))
    cfg2, get2 = KE.dir_source(str(tmp_path))  # the inner sizes of decay and gate come from the tensors' shapes
    assert cfg2.to_json() == cfg.to_json() and cfg2.layers[0].mlp is None and cfg2.layers[1].mlp.shared_ff is None
    assert cfg2.layers[2].mixer.rank_a == 3 and cfg2.layers[2].mixer.rank_g == 2 and cfg2.streams is None
    assert cfg2.bigram is None and cfg2.layers[0].mixer.rot_dims == 0 and cfg2.layers[1].mixer.rot_dims == 8
    assert torch.equal(get2("l1.mix.q"), get("l1.mix.q")) and get2("l0.hc1.in") is None and get2("bigram") is None
    from localai_tfp_amd.models.loader import load_llm
    m, _tok, c, _ = load_llm(str(tmp_path), "cpu")
    assert isinstance(m, KE.KeronexModel) and c.layers[1].mixer.scale == 0.4
    assert [sorted(e) for e in m.cache_spec()] == [["state"], ["kv"], ["state", "tails"], ["kv"]]
    cfg3 = KE.make_config(**SHAPES["plain"])  # streams, pair table, a layer on another's tensors
    j3 = cfg3.to_json()
    assert j3["streams"] == 3 and j3["layers"][3]["weights_of"] == 2 and "l3.norm1" not in KE.tensor_shapes(cfg3)
    assert KE.tensor_shapes(cfg3)["bigram"] == (62, 64) and KE.tensor_shapes(cfg3)["l0.hc2.mix"] == (3, 3)
    for L, L2 in zip(j3["layers"], cfg3.layers):
        if L["type"] == "channel_delta":
            L["mixer"].update(rank_a=L2.mixer.rank_a, rank_g=L2.mixer.rank_g)
    for path, val in ((("layers", 0, "type"), "something_else"), (("layers", 1, "mlp", "kind"), "glu"),
                      (("layers", 3, "weights_of"), 3), (("layers", 3, "weights_of"), 1), (("layers", 3, "mixer", "dim"), 8),
                      (("layers", 2, "mixer", "decay"), [0.5]), (("streams",), 33), (("layers", 0, "mixer", "kv_heads"), 3)):
        bad = json.loads(json.dumps(j3))
        KE.KeronexConfig.from_json(bad)  # (valid until it is broken)
        node = bad
        for p in path[:-1]:
            node = node[p]
        node[path[-1]] = val
        with pytest.raises(ValueError):
            KE.KeronexConfig.from_json(bad)
    tensors = {k: get(k) for k in get.names}
    tensors["l1.mix.q"] = tensors["l1.mix.q"][:-1]
    with pytest.raises(ValueError):
        KE.KeronexModel.load(cfg, tensors.get, "cpu")


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run on a checkpoint directory: steps on stdin, one logits file per step that wants any."""
    cfg = KE.make_config(**SHAPES["plain"])
    get = KE.synthetic_source(cfg, 6)
    mdir, odir = str(tmp_path / "m"), str(tmp_path / "o")
    KE.save_checkpoint(cfg, get, mdir)
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
    """The gRPC LLM worker loads a Keronex checkpoint directory like any other model and streams a completion whose
    tokens are the oracle's greedy continuation (byte-level tokenizer: one token per prompt byte after BOS)."""
    from localai_tfp_amd.grpc import pb
    from localai_tfp_amd.grpc.client import BackendClient
    from localai_tfp_amd.grpc.server import AioServer
    from localai_tfp_amd.workers.llm import LLMServicer
    cfg = KE.make_config(**dict(SHAPES["plain"], vocab=300))
    get = KE.synthetic_source(cfg, 12)
    KE.save_checkpoint(cfg, get, str(tmp_path))
    svc = LLMServicer(device="cpu")
    server = AioServer(svc, "127.0.0.1:0", max_workers=4)
    c = BackendClient(f"127.0.0.1:{server.port}")
    try:
        r = c.load_model(pb.ModelOptions(Model=str(tmp_path), ContextSize=256))
        assert r.success, r.message
        assert isinstance(svc.engine.model, KE.KeronexModel)
        o = pb.PredictOptions(Prompt="streams", Tokens=6, Temperature=0.0, IgnoreEOS=True)
        a = c.predict(o)
        chunks = list(c.predict_stream(o))
        assert a.tokens == 6 and b"".join(x.message for x in chunks) == a.message
        tok = svc.engine.tok
        seq = list(tok.encode("streams"))
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
