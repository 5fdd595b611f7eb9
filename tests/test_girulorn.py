"""Girulorn (sink attention with a distance bias, head norms, query temperature, head gates and borrowed keys, beside
gated linear attention with per-channel decays; expert feed-forwards; norms on the sublayers' outputs) on the engine
against the plain float64 oracle of tests/oracle_girulorn.py: every mechanism alone, whole prompts, token-by-token
decoding, prompt portions down to two tokens, unequal batches, reuse of freed blocks and state slots, keys far back / at
page borders / on both sides of a bias bucket's edge with peaked softmax weights, odd sizes, long decoding, greedy
generation through the scheduler, graph replays, and the trace runner's command line.

Each engine test runs on the CPU plumbing path (fp32) and, marked gpu, on the HIP kernels in fp32 and bf16."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import oracle_girulorn as O
from localai_tfp_amd.engine.engine import EngineConfig, LLMEngine
from localai_tfp_amd.models import girulorn as GI
from localai_tfp_amd.ops import hybrid as HY
from localai_tfp_amd.ops.sampling import SamplingParams
from localai_tfp_amd.tokenizer import ByteTokenizer
from test_vugotar import _FB, close, engine, run_cuts, steps_of, toks

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVS = ["cpu", GPU]
RUNS = [("cpu", "float32", 2e-4), pytest.param("cuda", "float32", 2e-4, marks=pytest.mark.gpu),
        pytest.param("cuda", "bfloat16", 6e-2, marks=pytest.mark.gpu)]

SHAPES = {
    # attention, gated linear attention, and an attention layer that reads the first one's keys and values
    "plain": dict(hidden=64, vocab=97, pattern=("attention", "gla", "attention"), kv_from={2: 0}, heads=4, kv_heads=2,
                  dim=16, vdim=16, bias_max=40.0, bias_rows=12, temp_coef=0.4, temp_every=8, g_heads=2, g_dim=16,
                  g_vdim=16, tau=4.0, rank=6, experts=4, top=2, expert_ff=32, shared_ff=32),
    # sizes that differ from each other: dim != vdim, as many key heads as heads, a bias table of two rows, no
    # temperature, top == experts, no shared expert, a layer without a feed-forward, a large eps, stacked projections
    # of odd total width, a borrowing layer right after a recurrent one, a recurrent first layer
    "odd": dict(hidden=40, vocab=61, pattern=("gla", "attention", "gla", "attention", "attention"), kv_from={3: 1, 4: 1},
                mlps=(None, "moe", "moe"), heads=3, kv_heads=3, dim=24, vdim=40, scale=0.4, bias_max=3.0, bias_rows=2,
                temp_coef=0.0, g_heads=3, g_dim=20, g_vdim=12, tau=1.0, rank=3, experts=5, top=5, expert_ff=17,
                shared_ff=0, eps=1e-3),
    # states wider than a lane keeps alone (160 numbers per column), value sizes that are no multiple of 64, one
    # expert of many, one key head for all heads, a temperature that steps at every position
    "wide": dict(hidden=48, vocab=53, pattern=("attention", "gla"), heads=4, kv_heads=1, dim=72, vdim=8, scale=0.2,
                 bias_max=1000.0, bias_rows=30, temp_coef=0.1, temp_every=1, g_heads=2, g_dim=160, g_vdim=80, tau=32.0,
                 rank=16, experts=9, top=1, expert_ff=16, shared_ff=24),
    # nothing a multiple of eight: width, vocabulary, head sizes, expert widths, the decay's inner size
    "ragged": dict(hidden=44, vocab=101, pattern=("gla", "attention"), heads=5, kv_heads=5, dim=20, vdim=12, scale=0.3,
                   bias_max=7.5, bias_rows=4, temp_coef=0.2, temp_every=3, g_heads=3, g_dim=10, g_vdim=6, tau=2.5,
                   rank=5, experts=3, top=2, expert_ff=10, shared_ff=6),
}


def build(device="cpu", dtype="float32", seed=0, **kw):
    cfg = GI.make_config(**kw)
    get = GI.synthetic_source(cfg, seed)
    model = GI.GirulornModel.load(cfg, get, torch.device(device), getattr(torch, dtype))
    return cfg, {k: get(k) for k in get.names}, model


def oracle(cfg, tensors, tokens, layers=None):
    return O.forward(cfg.to_json(), tensors.get, tokens, layers).float()


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
def test_output_norm_and_residual_add(dev):
    g = torch.Generator().manual_seed(1)
    eps = 0.3  # a large eps shows whether it sits inside the root
    for M, C in ((5, 72), (3, 1100), (2, 4500), (2, 17000)):  # the last is wider than a block keeps in registers
        y, x = torch.randn(M, C + 2, generator=g) * 3, torch.randn(M, C, generator=g)
        w = 1.0 + 0.2 * torch.randn(C, generator=g)
        want = x.double() + O.rms_norm(y[:, 2:].double(), w, eps)
        xd = x.clone().to(dev)
        o16 = torch.empty(M, C, device=dev, dtype=torch.bfloat16)
        HY.norm_add(y.to(dev)[:, 2:], w.to(dev), eps, xd, o16)
        close(xd, want, 1e-5)
        close(o16.float(), want, 1e-2)
        xd = x.clone().to(dev)
        HY.norm_add(y.to(dev)[:, 2:], (w - 1.0).to(dev), eps, xd, offset=1.0)  # a weight stored around one
        close(xd, want, 1e-5)


def test_distance_buckets():
    """One table row per distance: exact rows, logarithmic rows, everything from `far` on in the last row; whole
    logarithms (powers of two) fall on the upper side."""
    for rows, far in ((12, 40.0), (2, 3.0), (30, 1000.0), (32, 128.0), (64, 512.0), (8, 4.5), (16, 64.0)):
        rel = torch.arange(rows * 3, dtype=torch.float32).reshape(rows, 3)
        lut = HY.log_bucket_table(rel, far)
        assert lut.shape[1] >= far and lut.shape[0] == 3
        for n in range(lut.shape[1] + 20):
            assert lut[1, min(n, lut.shape[1] - 1)] == rel[O.distance_bucket(n, rows, far), 1], (rows, far, n)
    assert O.distance_bucket(64, 64, 512.0) == 40 and O.distance_bucket(63, 64, 512.0) == 39
    assert O.distance_bucket(127, 32, 128.0) == 31 and O.distance_bucket(10 ** 6, 32, 128.0) == 31


def _bias_attention_case(dev, dt, H, G, dk, dv, n, cuts, bs, scale, plant=(), rows=12, far=40.0, temp=(0.4, 8),
                         rel_scale=1.0, sink_shift=0.0):
    """Head norms + temperature + append, then attention with distance bias, learned sinks and head gates, in portions
    through shuffled pages. `plant` = [(query position, key position)]: the query is made parallel to the key, so
    that one score stands out."""
    g = torch.Generator().manual_seed(7)
    md = getattr(torch, dt)
    q = torch.randn(n, H * dk, generator=g)
    k = torch.randn(n, G * dk, generator=g)
    v = torch.randn(n, G * dv, generator=g)
    gate = torch.randn(n, H, generator=g) * 2
    qw, kw = 1.0 + 0.3 * torch.randn(dk, generator=g), 1.0 + 0.3 * torch.randn(dk, generator=g)
    rel = torch.randn(rows, H, generator=g) * rel_scale
    sink = torch.randn(H, generator=g) + sink_shift
    for qi, kj in plant:
        for h in range(H):  # every head's query points at key kj of its group (through both norm weights)
            gg = h // (H // G)
            q[qi, h * dk:(h + 1) * dk] = k[kj, gg * dk:(gg + 1) * dk] * kw / qw
    eps = 1e-6
    qd = O.rms_norm(q.double().reshape(n, H, dk), qw, eps)
    if temp:
        qd = qd * torch.tensor([O.query_temperature(p, *temp) for p in range(n)], dtype=torch.float64)[:, None, None]
    kd = O.rms_norm(k.double().reshape(n, G, dk), kw, eps)
    want = O.sink_bias_attention(qd, kd, v.double().reshape(n, G, dv), scale, rel, far, sink.double())
    want = (want * torch.sigmoid(gate.double())[:, :, None]).reshape(n, H * dv)
    lut = HY.log_bucket_table(rel, far).to(dev)
    nb = -(-n // bs)
    table = torch.randperm(nb + 3, generator=g)[:nb].tolist()  # pages out of order
    kc = torch.full((nb + 3, bs, G * dk), 7.0, dtype=md, device=dev)  # stale numbers in unused slots
    vc = torch.full((nb + 3, bs, G * dv), -5.0, dtype=md, device=dev)
    wide = torch.cat([torch.randn(n, 3, generator=g), q, k, v, gate], 1).to(dev)  # the projections as column slices
    got = torch.empty(n, H * dv + 5, device=dev, dtype=md)
    part = (torch.empty(H * 8, 2, device=dev), torch.empty(H * 8, dv, device=dev))  # room for eight partitions
    for n_dec, chunks, at in steps_of(n, cuts):
        c = 1 if n_dec else chunks[0]
        rws = list(range(at, at + c))
        slots = [table[p // bs] * bs + p % bs for p in rws]
        fb = _FB(n_dec, chunks, rws, [0], dev, slots, dec_bt=[table] if n_dec else None,
                 dec_lens=[at + 1] if n_dec else None, pf_bt=None if n_dec else [table],
                 pf_ctx=None if n_dec else [at + c])
        qo = torch.empty(c, H * dk, device=dev, dtype=md)
        w = wide[at:at + c]
        c0 = 3 + (H + G) * dk
        HY.rope_norm_append(w[:, 3:3 + H * dk], w[:, 3 + H * dk:c0], w[:, c0:c0 + G * dv], fb.positions, H, G, dk, dv, 0,
                            10.0, True, eps, qo, kc, vc, fb.slots, q_weight=qw.to(dev), k_weight=kw.to(dev), q_temp=temp)
        HY.masked_attention(qo, kc, vc, HY.Ragged(fb), H, G, dk, dv, scale, got[at:at + c, 5:], sink=sink.to(dev),
                            bias=lut, gate=w[:, c0 + G * dv:], out_scale=0.5, workspace=part)
    return got[:, 5:].float() * 2, want


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("gemm_rows", [64, 8])
def test_attention_bias_buckets_pages_sinks_and_gates(dev, dt, tol, gemm_rows, monkeypatch):
    """Planted keys carry nearly all the weight: far back beyond the table's last distance, across a page border, at
    the query's own position, at position 0; the bias table is scaled up so that a key on the wrong side of a bucket's
    edge moves the output. In prompt portions and in rows decoded alone; on the GPU portions of `gemm_rows` rows and
    more take the library-GEMM route (or the matrix cores), shorter ones and decoded rows the row kernels."""
    monkeypatch.setattr(HY, "GEMM_MIN_ROWS", gemm_rows)
    bs, n = 16, 150
    b16 = 4 if dt == "bfloat16" else 1
    plant = [(79, 40), (119, 80), (120, 119), (121, 120), (95, 81), (149, 12), (60, 60), (39, 0), (41, 39), (140, 100)]
    for cuts in ([n], [37, 2, 41, 1, 1, 38, 1, 1, 1, 27], [118] + [1] * 32):
        got, want = _bias_attention_case(dev, dt, 4, 2, 16, 24, n, cuts, bs, 4.0, plant, rel_scale=3.0)
        close(got, want, tol * b16)
    # one key head, sizes that are no multiple of eight, a table of two rows, no temperature, sinks that dominate
    got, want = _bias_attention_case(dev, dt, 3, 1, 12, 5, 70, [33, 2, 1, 1, 30, 3], 16, 0.7, rows=2, far=3.0, temp=None,
                                     sink_shift=4.0)
    close(got, want, tol)
    got, want = _bias_attention_case(dev, dt, 2, 2, 64, 72, 90, [50, 40], 8, 0.3, rows=30, far=1000.0, temp=(0.1, 1))
    close(got, want, tol)
    # head sizes of 64 and 128 (the matrix-core kernels take bf16 portions of 16 rows and more and decoded rows): four,
    # two and one query heads per key head, dim != vdim, portions that start and end inside 16-row tiles
    for H, G, dk, dv in ((4, 2, 64, 64), (8, 2, 128, 128), (2, 2, 64, 128), (6, 3, 128, 64), (5, 1, 64, 64)):
        got, want = _bias_attention_case(dev, dt, H, G, dk, dv, 150, [37, 2, 41, 1, 17, 22, 1, 29], bs, 0.5, plant,
                                         rel_scale=3.0)
        close(got, want, tol * b16)
    # rows decoded alone behind 260 and more visible keys: their keys are split into partitions and merged (the sink
    # and the gate join in the merge); the far keys lie beyond the bias table's last distance
    plant = [(270, 3), (280, 127), (281, 128), (299, 255), (290, 256), (295, 295)]
    got, want = _bias_attention_case(dev, dt, 2, 1, 16, 16, 300, [200, 60] + [1] * 40, 16, 3.0, plant, rel_scale=2.0)
    close(got, want, tol * b16)
    got, want = _bias_attention_case(dev, dt, 4, 1, 64, 64, 300, [200, 60] + [1] * 40, 16, 1.0, plant, rows=20, far=290.0)
    close(got, want, tol * b16)
    got, want = _bias_attention_case(dev, dt, 6, 2, 128, 64, 300, [259] + [1] * 41, 16, 0.5, plant, sink_shift=3.0)
    close(got, want, tol * b16)


@pytest.mark.gpu
def test_matrix_core_kernels_agree_with_the_row_kernels(monkeypatch):
    """bf16 runs round their operands, so the oracle bounds them only loosely; the matrix-core kernels (prompt portions,
    decoded rows, partitions) and the row kernels read the same rounded operands and must agree to a few bf16 steps: a
    wrong bias entry, sink or gate for any head would show at once."""
    plant = [(79, 40), (119, 80), (120, 119), (121, 120), (95, 81), (149, 12), (60, 60), (39, 0), (41, 39), (140, 100)]
    far = [(270, 3), (280, 127), (281, 128), (299, 255), (290, 256), (295, 295)]
    cases = [((H, G, dk, dv, 150, [37, 2, 41, 1, 17, 22, 1, 29], 16, 0.5, plant), {}) for H, G, dk, dv in
             ((4, 2, 64, 64), (8, 2, 128, 128), (2, 2, 64, 128), (6, 3, 128, 64), (5, 1, 64, 64), (16, 1, 64, 64))]
    cases += [((4, 1, 64, 64, 300, [200, 60] + [1] * 40, 16, 1.0, far), dict(rows=20, far=290.0)),
              ((7, 1, 128, 128, 300, [100, 100, 59] + [1] * 41, 16, 0.5, far), dict(sink_shift=1.0, rows=6, far=9.0))]
    for args, kw in cases:
        out = []
        for rows_min in (16, 0):  # 0: the matrix-core kernels are off
            monkeypatch.setattr(HY, "MFMA_MIN_ROWS", rows_min)
            got, want = _bias_attention_case("cuda", "bfloat16", *args, rel_scale=3.0, **kw)
            out.append(got.double().cpu())
        assert (out[0] - out[1]).abs().max().item() < 0.04, args[:4]  # values of up to 4: 1/64 is one bf16 step
        close(out[0], want, 0.06)


@pytest.mark.parametrize("dev", DEVS)
def test_learned_sink_takes_or_leaves_the_weight(dev):
    """A large sink score holds the denominator (outputs shrink towards zero), a very negative one leaves the plain
    softmax; a closed gate silences its head only."""
    n, dk, dv, H = 6, 8, 8, 2
    g = torch.Generator().manual_seed(3)
    q = torch.randn(n, H * dk, generator=g)
    outs = []
    for sink, gate in (([30.0, -30.0], None), ([-30.0, -30.0], [[-40.0, 0.0]] * n)):
        kc, vc = torch.zeros(2, 8, dk, device=dev), torch.zeros(2, 8, dv, device=dev)
        fb = _FB(0, [n], list(range(n)), [0], dev, list(range(n)), pf_bt=[[0, 1]], pf_ctx=[n])
        qo = torch.empty(n, H * dk, device=dev)
        HY.rope_norm_append(q.to(dev), q[:, :dk].contiguous().to(dev), torch.ones(n, dv, device=dev), fb.positions, H, 1,
                            dk, dv, 0, 10.0, True, 1e-6, qo, kc, vc, fb.slots)
        o = torch.empty(n, H * dv, device=dev)
        HY.masked_attention(qo, kc, vc, HY.Ragged(fb), H, 1, dk, dv, 1.0, o, sink=torch.tensor(sink, device=dev),
                            gate=None if gate is None else torch.tensor(gate, device=dev))
        outs.append(o.cpu())
    assert outs[0][:, :dv].abs().max() < 1e-6 and torch.allclose(outs[0][:, dv:], torch.ones(n, dv), atol=1e-5)
    assert outs[1][:, :dv].abs().max() < 1e-6 and torch.allclose(outs[1][:, dv:], 0.5 * torch.ones(n, dv), atol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("H,N,P", [(2, 16, 16), (3, 20, 12), (2, 160, 80), (1, 128, 128), (3, 48, 72), (2, 256, 8)])
def test_channel_decay_scan_in_portions(dev, H, N, P):
    g = torch.Generator().manual_seed(N + P)
    n, tau = 45, 3.0
    k = torch.randn(n, H * N, generator=g)
    q = torch.randn(n, H * N + 2, generator=g)
    v = torch.randn(n, H * P, generator=g)
    z, zb = torch.randn(n, H * N, generator=g) * 3, torch.randn(H * N, generator=g)
    z[5, :4] = -60.0  # log_sigmoid without overflow: a channel that forgets everything
    z[6, :4] = 60.0
    alpha = torch.sigmoid(z.double() + zb.double()).pow(1.0 / tau)
    want = O.channel_decay_recurrence(q[:, 2:].double().reshape(n, H, N) * N ** -0.5, k.double().reshape(n, H, N),
                                      v.double().reshape(n, H, P), alpha.reshape(n, H, N)).reshape(n, H * P)
    dec = torch.empty(n, H * N, device=dev)
    HY.channel_decay(z.to(dev), zb.to(dev), tau, dec)
    close(dec, alpha, 1e-5)
    for R in (3, 16, 300):  # the same with the second half of a low-rank projection inside
        lo, pr = torch.randn(n, R + 1, generator=g), torch.randn(R, H * N, generator=g) * R ** -0.5
        dec2 = torch.empty(n, H * N, device=dev)
        HY.channel_decay(lo.to(dev)[:, 1:], zb.to(dev), tau, dec2, proj=pr.to(dev))
        close(dec2, torch.sigmoid(lo[:, 1:].double() @ pr.double() + zb.double()).pow(1.0 / tau), 1e-5)
    state = torch.full((2, H, P, N), 4.0, device=dev)  # slot 1 is dirty: position 0 must not read it
    out = torch.empty(n, H * P, device=dev)
    for n_dec, chunks, at in steps_of(n, [9, 1, 2, 1, 1, 20, 3, 2, 1, 5]):
        c = 1 if n_dec else chunks[0]
        fb = _FB(n_dec, chunks, list(range(at, at + c)), [1], dev)
        sl = slice(at, at + c)
        HY.state_scan(k.to(dev)[sl], q.to(dev)[sl, 2:], v.to(dev)[sl], dec[sl], None, None, state, HY.Ragged(fb), out[sl],
                      H, H, N, P, delta=False, channel=True, q_scale=N ** -0.5)
    close(out, want, 2e-5)
    assert float(state[0].min()) == 4.0  # the other slot is untouched
    # a decode row of one sequence beside a fresh chunk of another that takes over a dirty slot
    st2 = torch.full((2, H, P, N), -2.0, device=dev)
    first = torch.empty(5, H * P, device=dev)
    HY.state_scan(k.to(dev)[:5], q.to(dev)[:5, 2:], v.to(dev)[:5], dec[:5], None, None, st2,
                  HY.Ragged(_FB(0, [5], list(range(5)), [1], dev)), first, H, H, N, P, delta=False, channel=True,
                  q_scale=N ** -0.5)
    idx = [5] + list(range(6))
    both = torch.empty(7, H * P, device=dev)
    HY.state_scan(k.to(dev)[idx], q.to(dev)[idx][:, 2:], v.to(dev)[idx], dec[idx].contiguous(), None, None, st2,
                  HY.Ragged(_FB(1, [6], idx, [1, 0], dev)), both, H, H, N, P, delta=False, channel=True,
                  q_scale=N ** -0.5)
    close(both[0], want[5], 2e-5)
    close(both[1:], want[:6], 2e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_router_softmax_over_the_chosen_logits(dev):
    g = torch.Generator().manual_seed(5)
    T = 6
    for E, top in ((7, 3), (5, 5), (70, 1), (130, 4), (8, 4)):
        z, b = torch.randn(T, E + 1, generator=g) * 2, torch.randn(E, generator=g) * 2
        z[0, 1:] += 80.0  # large logits: nothing overflows
        wts = torch.empty(T, E, device=dev)
        HY.moe_route(z.to(dev)[:, 1:], top, 1.0, wts, 0.0, bias=b.to(dev))
        zz = z[:, 1:].double() + b.double()
        tv, ti = torch.topk(zz, top, -1)
        want = torch.zeros(T, E, dtype=torch.float64).scatter_(1, ti, torch.softmax(tv, -1))
        close(wts, want, 1e-5)


# ------------------------------------------------------------------------------------------------ whole model
@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("shape", list(SHAPES))
def test_prompt_portions_and_decoding(dev, dt, tol, shape):
    """The whole prompt in one step, token-by-token decoding after a prefix, and portions of several sizes down to
    two tokens (cut inside pages and bias buckets): all give the oracle's logits."""
    cfg, tensors, model = build(dev, dt, seed=3, **SHAPES[shape])
    t = toks(75, cfg.vocab, 5)
    want = oracle(cfg, tensors, t)
    eng = engine(model, 96)
    b16 = dt == "bfloat16"  # (the sublayers read the residual itself, rounded to bf16: no norm in front of them)
    if b16 and shape in ("odd", "ragged"):  # some 40 numbers wide: single rows carry several times the typical rounding
        tol *= 2
    close(run_cuts(eng, "whole", t, [75]), want, tol, b16)
    close(run_cuts(eng, "decode", t, [40] + [1] * 35), want, tol, b16)
    close(run_cuts(eng, "cuts", t, [3, 2, 19, 2, 1, 1, 30, 2, 7, 1, 1, 1, 5]), want, tol, b16)
    close(run_cuts(eng, "first", t[:9], [1] * 9), want[:9], tol, b16)  # the first tokens, one by one from position 0
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 4


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("kind", ["gla", "attention"])
def test_models_of_one_kind_of_layer(dev, dt, tol, kind):
    """Recurrent layers only (the paged pool is empty, blocks are bookkeeping) and attention layers only (the state
    slots hold nothing), the second with a table of an odd number of rows and no feed-forward anywhere."""
    kw = dict(SHAPES["plain"], pattern=(kind,) * 3, kv_from={2: 1} if kind == "attention" else None)
    if kind == "attention":
        kw.update(mlps=(None,), bias_rows=7, bias_max=11.0)
    cfg, tensors, model = build(dev, dt, seed=13, **kw)
    assert (model.cache_ranks() == []) == (kind == "gla")
    t = toks(60, cfg.vocab, 3)
    want = oracle(cfg, tensors, t)
    ec = EngineConfig(max_num_seqs=2, max_batched_tokens=64, max_model_len=64, block_size=16, use_graphs=False,
                      overlap=False, native_scheduler=False, logits_rows=64, gemm_autotune=False,
                      num_blocks=0 if kind == "gla" else 9)
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
        close(torch.cat(got[k]), want[k], tol, dt == "bfloat16")
        # and the same request alone, in the same number format: no router tie falls differently here
        alone = run_cuts(eng, "alone-" + k, reqs[k], [len(reqs[k])])
        close(torch.cat(got[k]), alone, 2e-4 if dt == "float32" else 4e-3)
    assert eng.bm.num_free == eng.bm.num_blocks - 1 and len(eng.state_slots.free) == 3


@pytest.mark.parametrize("dev,dt,tol", RUNS)
def test_peaked_attention_far_keys_and_long_decode(dev, dt, tol):
    """A large score scale makes single keys dominate, so a lost or shifted key anywhere in a long prompt (page
    borders, position 0, beyond the bias table's last distance) moves the logits; then 70 tokens decoded one by one
    while the temperature steps and the decayed state is carried on."""
    kw = dict(SHAPES["plain"], scale=2.5, bias_max=100.0, temp_every=50)
    cfg, tensors, model = build(dev, dt, seed=21, **kw)
    t = toks(260, cfg.vocab, 8)
    want = oracle(cfg, tensors, t)
    eng = engine(model, max_tokens=272, seqs=2)
    got = run_cuts(eng, "x", t, [187, 3] + [1] * 70)
    close(got, want, tol * 2, rms=dt == "bfloat16")


@pytest.mark.parametrize("dev,dt,tol", RUNS)
@pytest.mark.parametrize("dim,vdim,heads,kv", [(64, 128, 8, 2), (128, 64, 3, 1), (64, 64, 20, 1)])
def test_matrix_core_head_sizes_through_the_engine(dev, dt, tol, dim, vdim, heads, kv):
    """Head sizes of 64 / 128 (bf16 prompts and decoded rows run on the matrix cores, up to 16 query heads per key
    head; 20 take the row kernel): a prompt longer than the bias table, portions that end inside 16-row tiles, decoded
    rows behind enough keys to be split into partitions, a borrowing layer."""
    kw = dict(hidden=128, vocab=211, pattern=("attention", "gla", "attention"), kv_from={2: 0}, heads=heads, kv_heads=kv,
              dim=dim, vdim=vdim, scale=1.5 * dim ** -0.5, bias_max=200.0, bias_rows=16, temp_coef=0.3, temp_every=100,
              g_heads=2, g_dim=64, g_vdim=64, tau=8.0, rank=4, experts=4, top=2, expert_ff=64, shared_ff=64)
    cfg, tensors, model = build(dev, dt, seed=17, **kw)
    t = toks(330, cfg.vocab, 9)
    want = oracle(cfg, tensors, t)
    eng = engine(model, max_tokens=336, seqs=2)
    b16 = dt == "bfloat16"
    close(run_cuts(eng, "x", t, [203, 17, 2, 41, 1, 1, 1, 33] + [1] * 31), want, tol, b16)
    close(run_cuts(eng, "y", t[:100], [100]), want[:100], tol, b16)


def _random_shape(rng):
    nl = rng.randint(2, 6)
    pattern, kv_from, owners = [], {}, []
    for i in range(nl):
        kind = rng.choice(["attention", "gla"])
        pattern.append(kind)
        if kind == "attention":
            if owners and rng.random() < 0.4:
                kv_from[i] = rng.choice(owners)
            else:
                owners.append(i)
    kv, rows, experts = rng.choice([1, 2, 3, 4]), rng.choice([2, 4, 8, 16, 32, 64]), rng.choice([2, 3, 4, 8, 16])
    return dict(hidden=rng.choice([64, 96, 160]), vocab=rng.choice([97, 256, 1000]), pattern=tuple(pattern),
                kv_from=kv_from, heads=kv * rng.choice([1, 2, 3, 6]), kv_heads=kv, dim=rng.choice([16, 32, 48, 64, 128]),
                vdim=rng.choice([16, 32, 64, 128]), scale=rng.choice([0.05, 0.1, 0.2]),
                bias_max=float(max(rows // 2 + 1, rng.choice([3, 30, 120, 500]))), bias_rows=rows,
                temp_coef=rng.choice([0.0, 0.1, 0.5]), temp_every=rng.choice([1, 7, 64]), g_heads=rng.choice([1, 2, 4]),
                g_dim=rng.choice([16, 32, 48, 64, 128]), g_vdim=rng.choice([16, 32, 96]), tau=rng.choice([1.0, 4.0, 64.0]),
                rank=rng.choice([1, 4, 16]), mlps=tuple(rng.choice(["moe", "moe", None]) for _ in range(rng.randint(1, 3))),
                experts=experts, top=rng.randint(1, experts), expert_ff=rng.choice([16, 40]),
                shared_ff=rng.choice([0, 32, 96]), eps=rng.choice([1e-6, 1e-5]))


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_configurations_and_schedules(dev, seed):
    """Drawn sizes, layer orders and borrowings; five requests fed through four live slots in drawn portions (single
    tokens beside portions of up to 150, requests left out of steps, blocks and slots handed on) in a pool that holds
    the four largest but not all five. fp32 only: every position agrees with the oracle."""
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
    cfg = GI.make_config(**SHAPES["odd"])
    get = GI.synthetic_source(cfg, 1)
    GI.save_checkpoint(cfg, get, str(tmp_path))
    assert GI.is_girulorn_dir(str(tmp_path))
    cfg2, get2 = GI.dir_source(str(tmp_path))  # table rows and the decay's inner size come from the tensors' shapes
    assert cfg2.to_json() == cfg.to_json() and cfg2.layers[0].mlp is None and cfg2.layers[1].mlp.shared_ff is None
    assert cfg2.layers[1].mixer.bias_rows == 2 and cfg2.layers[0].mixer.rank == 3 and cfg2.layers[4].mixer.kv_from == 1
    assert torch.equal(get2("l1.mix.q"), get("l1.mix.q")) and get2("l3.mix.k") is None and get2("l0.mlp.router") is None
    from localai_tfp_amd.models.loader import load_llm
    m, _tok, c, _ = load_llm(str(tmp_path), "cpu")
    assert isinstance(m, GI.GirulornModel) and c.layers[1].mixer.scale == 0.4
    assert [bool(e.get("kv")) for e in m.cache_spec()] == [False, True, False, False, False]
    for path, val in ((("layers", 0, "type"), "something_else"), (("layers", 1, "mlp", "kind"), "dense"),
                      (("layers", 3, "mixer", "kv_from"), 2), (("layers", 3, "mixer", "kv_from"), 4),
                      (("layers", 4, "mixer", "dim"), 16)):
        bad = cfg2.to_json()
        for L, L2 in zip(bad["layers"], cfg2.layers):
            if L["type"] == "attention":
                L["mixer"]["bias_rows"] = L2.mixer.bias_rows
            else:
                L["mixer"]["rank"] = L2.mixer.rank
        GI.GirulornConfig.from_json(bad)  # (valid until it is broken)
        node = bad
        for p in path[:-1]:
            node = node[p]
        node[path[-1]] = val
        with pytest.raises(ValueError):
            GI.GirulornConfig.from_json(bad)
    tensors = {k: get(k) for k in get.names}
    tensors["l1.mix.q"] = tensors["l1.mix.q"][:-1]
    with pytest.raises(ValueError):
        GI.GirulornModel.load(cfg, tensors.get, "cpu")


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run on a checkpoint directory: steps on stdin, one logits file per step that wants any."""
    cfg = GI.make_config(**SHAPES["plain"])
    get = GI.synthetic_source(cfg, 6)
    mdir, odir = str(tmp_path / "m"), str(tmp_path / "o")
    GI.save_checkpoint(cfg, get, mdir)
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
    """The gRPC LLM worker loads a Girulorn checkpoint directory like any other model and streams a completion whose
    tokens are the oracle's greedy continuation (byte-level tokenizer: one token per prompt byte after BOS)."""
    from localai_tfp_amd.grpc import pb
    from localai_tfp_amd.grpc.client import BackendClient
    from localai_tfp_amd.grpc.server import AioServer
    from localai_tfp_amd.workers.llm import LLMServicer
    cfg = GI.make_config(**dict(SHAPES["plain"], vocab=300))
    get = GI.synthetic_source(cfg, 12)
    GI.save_checkpoint(cfg, get, str(tmp_path))
    svc = LLMServicer(device="cpu")
    server = AioServer(svc, "127.0.0.1:0", max_workers=4)
    c = BackendClient(f"127.0.0.1:{server.port}")
    try:
        r = c.load_model(pb.ModelOptions(Model=str(tmp_path), ContextSize=256))
        assert r.success, r.message
        assert isinstance(svc.engine.model, GI.GirulornModel)
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
