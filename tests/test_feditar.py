"""Feditar (mLSTM / Mamba-2 / parallel attention + decayed-memory
decoder) against a plain float64 model written from the equations
(tests/feditar_oracle.py).

Every test builds its own small configuration and random checkpoint; the
engine reads it through the product loader.  Device-parametrized: the CPU
cases run the reference ops, the GPU cases the HIP kernels, both through
the same engine, cache manager and scheduler.
"""
import math
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import feditar_oracle as oracle
from inference_gateway_amd import ops
from inference_gateway_amd.engine.config import (EngineConfig,
                                                 FeditarConfig,
                                                 SamplingParams)
from inference_gateway_amd.engine.engine import LLMEngine
from inference_gateway_amd.engine.models.registry import (
    is_recurrent, model_config_from_dir)

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def _dev(device):
    return "cuda:0" if device == "cuda" else "cpu"


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def f32(x, device):
    return torch.tensor(np.asarray(x), dtype=torch.float32, device=device)


# four configurations; sizes all differ from one another
def cfg_small():
    return oracle.make_config(40, 61, [
        oracle.mlstm_layer(2, 6, 5),
        oracle.mamba2_layer(4, 5, 7, 2, 3, 2),
        oracle.parallel_layer(4, 2, 6, 9, 3, 0.3, 4, 0.3, 5.0, 2, 10,
                              ff=24),
        oracle.mlstm_layer(1, 9, 4, cap=6.0)])


def cfg_ones():
    """Single heads and groups, one norm part, two taps, a query stretch
    that changes at every position, no squashing to speak of, a mixer
    order that starts with the parallel pair."""
    return oracle.make_config(24, 37, [
        oracle.parallel_layer(1, 1, 5, 3, 2, 0.5, 1, 0.45, 50.0, 1, 4),
        oracle.mamba2_layer(1, 6, 3, 1, 2, 1, ff=16),
        oracle.mlstm_layer(1, 3, 7, cap=20.0, ff=12),
        oracle.parallel_layer(3, 3, 4, 4, 4, 0.0, 7, 0.5, 2.0, 3, 2)],
        buckets=11, mul_prev=1, mul_cur=1, scale=1.0, eps=1e-6)


def cfg_wide():
    """Widths that straddle the kernels' tile sizes: more than 64 value
    entries per head, key widths off the powers of two, many heads on
    one key/value head."""
    return oracle.make_config(72, 83, [
        oracle.mamba2_layer(6, 11, 17, 3, 4, 3),
        oracle.mlstm_layer(2, 33, 70),
        oracle.parallel_layer(6, 1, 20, 66, 5, 0.2, 16, 0.22, 8.0, 4, 18,
                              ff=40)],
        buckets=53, mul_prev=13, mul_cur=29)


CONFIGS = {"small": cfg_small, "ones": cfg_ones, "wide": cfg_wide}


def make_engine(tmp_path, cfg, W, device, dtype="float32", blocks=48,
                block=4, slots=4, **kw):
    path = oracle.save_checkpoint(Path(tmp_path) / "ckpt", cfg, W)
    ecfg = EngineConfig(
        model=model_config_from_dir(path), block_size=block,
        num_gpu_blocks=blocks, max_num_seqs=slots,
        max_batched_tokens=kw.pop("max_batched_tokens", 4096),
        max_model_len=cfg["max_positions"], use_hip_graphs=False,
        weights_path=path, dtype=dtype, **kw)
    return LLMEngine(ecfg, device=_dev(device))


def close(got, ref, tol):
    """Mean-free relative RMS difference per row, like a logit check."""
    got = torch.as_tensor(np.asarray(got.cpu() if torch.is_tensor(got)
                                     else got)).double()
    ref = torch.as_tensor(np.asarray(ref)).double()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()
    assert float(err.max()) < tol, f"rel err {float(err.max()):.3e}"


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay_all(engine, tokens, cuts):
    """Feed one request in portions `cuts`; logits of every position."""
    sid = engine.open_stream()
    out, at = [], 0
    for n in cuts:
        part = tokens[at:at + n]
        out.append(engine.replay_step([(sid, part)],
                                      {sid: list(range(len(part)))}))
        at += n
    assert at == len(tokens)
    engine.close_stream(sid)
    return torch.cat(out)


def ragged(rows, starts, slots, device):
    cu = [0]
    for n in rows:
        cu.append(cu[-1] + n)
    row_seq = [s for s, n in enumerate(rows) for _ in range(n)]
    return (i32(cu, device), i32(starts, device), i32(slots, device),
            i32(row_seq, device), cu)


# ---------------------------------------------------------------------------
# mechanisms alone: each op in two steps (a fresh portion, then a
# continued one) against the oracle run over the whole sequence
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_embedding_pair_hash_and_slots(device):
    cfg = oracle.make_config(20, 31, [], buckets=13, mul_prev=5, mul_cur=11,
                             scale=3.0, max_positions=64)
    W = oracle.random_weights(cfg, 1)
    seqs = [toks(9, 31, 2), toks(5, 31, 3), toks(1, 31, 4)]
    ref = [oracle.embed(t, W, cfg, 1e-5) for t in seqs]
    tab = {k: f32(W[k], device) for k in ("embed", "bigram", "pos")}
    w = f32(1.0 + W["embed.norm"], device)
    prev = torch.full((6, 1), 7, dtype=torch.int32, device=device)  # stale
    slots = [4, 0, 2]
    for step, cuts in enumerate([(4, 2, 1), (5, 3, 0)]):
        rows, starts, sl, tk, ps, want = [], [], [], [], [], []
        for s, seq in enumerate(seqs):
            a = 0 if step == 0 else (4, 2, 1)[s]
            n = cuts[s]
            if n == 0:
                continue
            rows.append(n), starts.append(a), sl.append(slots[s])
            tk += seq[a:a + n]
            ps += list(range(a, a + n))
            want.append(ref[s][a:a + n])
        cu, st, so, rs, _ = ragged(rows, starts, sl, device)
        out = ops.embed_pair_norm(
            torch.tensor(tk, dtype=torch.int64, device=device),
            i32(ps, device), prev, cu, st, so, rs, tab["embed"],
            tab["bigram"], tab["pos"], w, 3.0, 13, 5, 11, 1e-5)
        np.testing.assert_allclose(out.cpu().numpy(), np.concatenate(want),
                                   atol=2e-5, rtol=2e-5)
    assert prev[:, 0].tolist() == [seqs[1][4], 7, seqs[2][0], 7,
                                   seqs[0][8], 7]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("silu", [False, True])
@pytest.mark.parametrize("C", [70, 72])
def test_causal_conv_portions(device, taps, silu, C):
    """Portions shorter than the filter, a one-row continuation and a
    fresh sequence over stale history; strided input rows."""
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g) if silu else None
    full = [torch.randn(n, C + 8, generator=g) for n in (11, 6, 3)]
    ref = []
    for x in full:
        y = oracle.short_conv(x[:, :C].double().numpy(), w.double().numpy(),
                              None if b is None else b.double().numpy())
        ref.append(oracle.silu(y) if silu else y)
    state = torch.randn(5, max(1, (taps - 1) * C), generator=g).to(device)
    slots = [3, 1, 4]
    plans = [[(0, 2), (0, 6), (0, 1)], [(2, 1), None, (1, 2)],
             [(3, 8), None, None]]
    for plan in plans:
        rows, starts, sl, xs, want = [], [], [], [], []
        for s, pl in enumerate(plan):
            if pl is None:
                continue
            a, n = pl
            rows.append(n), starts.append(a), sl.append(slots[s])
            xs.append(full[s][a:a + n])
            want.append(ref[s][a:a + n])
        cu, st, so, rs, _ = ragged(rows, starts, sl, device)
        x = torch.cat(xs).to(device)
        out = ops.causal_conv(x[:, :C], w.to(device),
                              None if b is None else b.to(device), state,
                              cu, st, so, rs, silu)
        np.testing.assert_allclose(out.cpu().numpy(), np.concatenate(want),
                                   atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_mix(device):
    D = 37
    g = torch.Generator().manual_seed(5)
    mu = torch.rand(5, D, generator=g)
    full = [torch.randn(n, D, generator=g) for n in (7, 4)]
    state = torch.randn(4, D, generator=g).to(device)
    for plan in ([(0, 3), (0, 1)], [(3, 1), (1, 3)], [(4, 3), None]):
        rows, starts, sl, hs, want = [], [], [], [], []
        for s, pl in enumerate(plan):
            if pl is None:
                continue
            a, n = pl
            rows.append(n), starts.append(a), sl.append([2, 0][s])
            h = full[s].double()
            prev = torch.cat([torch.zeros(1, D).double(), h[:-1]])
            hs.append(full[s][a:a + n])
            want.append((h[None] + (prev - h)[None]
                         * mu.double()[:, None])[:, a:a + n])
        cu, st, so, rs, _ = ragged(rows, starts, sl, device)
        out = ops.token_shift_mix(torch.cat(hs).to(device), mu.to(device),
                                  state, cu, st, so, rs)
        np.testing.assert_allclose(out.cpu().numpy(),
                                   torch.cat(want, 1).numpy(), atol=1e-5,
                                   rtol=1e-5)


def _scan_reference(q, k, v, a, c, u, skip, ones, qscale):
    """float64 loop over one sequence: q, k [T, G, N], v [T, H, P], a
    [T, H, N|1], c [T, H] or None."""
    T, H, P = v.shape
    G, N = q.shape[1:]
    if ones:
        v = np.concatenate([v, np.ones((T, H, 1))], 2)
    S = np.zeros((H, N, v.shape[2]))
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            kk = k[t, g] * (1.0 if c is None else c[t, h])
            kv = np.outer(kk, v[t, h])
            at = np.broadcast_to(a[t, h], (N,))[:, None]
            if u is None:
                S[h] = at * S[h] + kv
                out[t, h] = S[h].T @ q[t, g]
            else:
                out[t, h] = (S[h] + u[h][:, None] * kv).T @ q[t, g]
                S[h] = at * S[h] + kv
    out = out * qscale
    if skip is not None:
        out[:, :, :P] += skip[None, :, None] * v[:, :, :P]
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [
    # H, G, N, P, form
    (2, 2, 6, 5, "mlstm"), (4, 2, 17, 3, "ssm"), (3, 3, 10, 10, "decay"),
    (2, 1, 33, 70, "mlstm"), (1, 1, 130, 65, "ssm"), (2, 2, 70, 70, "decay"),
    (1, 1, 1, 1, "ssm"), (2, 2, 8, 200, "mlstm"), (2, 1, 64, 300, "ssm"),
    (2, 2, 32, 64, "decay"), (1, 1, 128, 16, "mlstm")])
def test_outer_scan_forms(device, shape):
    """The three uses of the memory kernel, in two steps over a ragged
    batch: a fresh sequence in a stale slot, a continued one, a long one
    (several staged chunks) and a single row."""
    H, G, N, P, form = shape
    g = torch.Generator().manual_seed(N * 7 + P)
    lens = [45, 9, 2]
    data = []
    for T in lens:
        q = torch.randn(T, G, N, generator=g) * N ** -0.25
        k = torch.randn(T, G, N, generator=g) * N ** -0.25
        v = torch.randn(T, H, P, generator=g)
        if form == "decay":
            x = torch.randn(T, H, N, generator=g) * 0.7 - 1.0
            a, c = torch.exp(-torch.exp(x)), None
            dec = x
        else:
            a = torch.rand(T, H, 1, generator=g) * 0.5 + 0.5
            c = torch.rand(T, H, generator=g) + 0.2
            dec = a
        data.append((q, k, v, a, c, dec))
    u = torch.randn(H, N, generator=g) if form == "decay" else None
    skip = torch.randn(H, generator=g) if form == "ssm" else None
    ones = form == "mlstm"
    qscale = 0.37 if form == "mlstm" else 1.0
    refs = [_scan_reference(
        q.double().numpy(), k.double().numpy(), v.double().numpy(),
        a.double().numpy(), None if c is None else c.double().numpy(),
        None if u is None else u.double().numpy(),
        None if skip is None else skip.double().numpy(), ones, qscale)
        for q, k, v, a, c, dec in data]
    PP = P + (1 if ones else 0)
    state = torch.randn(4, H * N * PP, generator=g).to(device)
    slots = [1, 3, 0]
    for plan in ([(0, 40), (0, 1), (0, 2)], [(40, 5), (1, 8), None]):
        rows, starts, sl, parts, want = [], [], [], [], []
        for s, pl in enumerate(plan):
            if pl is None:
                continue
            a0, n = pl
            rows.append(n), starts.append(a0), sl.append(slots[s])
            parts.append([x[a0:a0 + n] if x is not None else None
                          for x in data[s]])
            want.append(refs[s][a0:a0 + n])
        cu, st, so, rs, _ = ragged(rows, starts, sl, device)
        cat = [torch.cat([p[i] for p in parts]).to(device)
               if parts[0][i] is not None else None for i in range(6)]
        out, nrm = ops.outer_scan(
            cat[0], cat[1], cat[2], cat[5].contiguous(), cat[4],
            None if u is None else u.to(device),
            None if skip is None else skip.to(device), state, cu, st, so,
            rows, ops.DECAY_EXP_NEG_EXP if form == "decay"
            else ops.DECAY_LINEAR, ones, qscale)
        want = np.concatenate(want)
        np.testing.assert_allclose(out.cpu().numpy(), want[:, :, :P],
                                   atol=2e-4, rtol=2e-4)
        if ones:
            np.testing.assert_allclose(nrm.cpu().numpy(), want[:, :, P],
                                       atol=2e-4, rtol=2e-4)
        else:
            assert nrm is None


@pytest.mark.parametrize("device", DEVICES)
def test_mlstm_gates_running_maximum(device):
    """The maximum starts at zero, not below: small input gates at the
    start must not lift it; a continued sequence resumes from its slot."""
    H, cap = 3, 4.0
    g = torch.Generator().manual_seed(6)
    pre = torch.randn(12, 2 * H, generator=g) * 3
    pre[:3, :H] = -9.0                       # tiny input gates first
    gi = cap * np.tanh(pre[:, :H].double().numpy() / cap)
    gf = oracle.logsigmoid(cap * np.tanh(pre[:, H:].double().numpy() / cap))
    m = np.zeros(H)
    ref = []
    for t in range(12):
        mn = np.maximum(gf[t] + m, gi[t])
        ref.append((np.exp(gf[t] + m - mn), np.exp(gi[t] - mn), np.exp(-mn)))
        m = mn
    assert ref[0][2].min() >= 1.0 - 1e-12     # exp(-m) with m <= 0
    ms = torch.full((3, H), 5.0, device=device)
    outs = []
    for a, n in ((0, 5), (5, 7)):
        cu, st, so, rs, _ = ragged([n], [a], [1], device)
        outs.append(torch.stack(ops.mlstm_gates(
            pre[a:a + n].to(device), cap, ms, cu, st, so)))
    got = torch.cat(outs, 1).cpu().numpy()
    for j in range(3):
        np.testing.assert_allclose(got[j], np.stack([r[j] for r in ref]),
                                   atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(ms[1].cpu().numpy(), m, atol=1e-5)
    assert ms[0].tolist() == [5.0] * H


@pytest.mark.parametrize("device", DEVICES)
def test_head_norm_gate_modes(device):
    g = torch.Generator().manual_seed(7)
    T, H, P = 5, 4, 6
    o = torch.randn(T, H, P + 1, generator=g)
    o[0, 0, P] = 1e-4                       # the floor decides here
    gate = torch.randn(T, H * P + 2, generator=g)
    w = torch.randn(H * P, generator=g)
    floor = torch.rand(T, H, generator=g) + 0.1
    od, gd, fd = (o.double().numpy(), gate[:, :H * P].double().numpy(),
                  floor.double().numpy())
    # normaliser division, per-head norm, sigmoid gate after
    den = np.maximum(np.abs(od[:, :, P]), fd) + 1e-6
    ref = oracle.rms_unit(od[:, :, :P] / den[:, :, None], 1e-5).reshape(
        T, -1) * w.double().numpy() * oracle.sigmoid(gd)
    got = ops.head_norm_gate(o[:, :, :P].contiguous().to(device),
                             gate[:, :H * P].to(device), w.to(device), 1e-5,
                             P, ops.GATE_SIGMOID, False,
                             o[:, :, P].contiguous().to(device),
                             floor.to(device), torch.float32)
    np.testing.assert_allclose(got.cpu().numpy(), ref, atol=2e-5, rtol=2e-5)
    # silu gate first, norm in two parts that span heads
    o2 = o[:, :, :P].contiguous()
    y = o2.double().numpy().reshape(T, -1) * oracle.silu(gd)
    ref = oracle.rms_unit(y.reshape(T, 2, -1), 1e-5).reshape(T, -1) \
        * w.double().numpy()
    got = ops.head_norm_gate(o2.to(device), gate[:, :H * P].to(device),
                             w.to(device), 1e-5, H * P // 2, ops.GATE_SILU,
                             True, None, None, torch.float32)
    np.testing.assert_allclose(got.cpu().numpy(), ref, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(3, 5, 130, 650), (2, 4, 96, 384),
                                  (4, 3, 70, 70), (3, 2, 128, 128),
                                  (2, 8, 128, 1024), (2, 9, 128, 1152)])
def test_head_norm_gate_group_sizes(device, dims):
    """Groups from one head to several, up to the two-pass kernel."""
    T, H, P, group = dims
    g = torch.Generator().manual_seed(P)
    o = torch.randn(T, H, P, generator=g)
    gate = torch.randn(T, H * P, generator=g)
    w = torch.randn(H * P, generator=g)
    for first in (True, False):
        y = o.double().numpy().reshape(T, -1)
        a = oracle.silu(gate.double().numpy())
        if first:
            y = y * a
        y = oracle.rms_unit(y.reshape(T, -1, group), 1e-6).reshape(T, -1) \
            * w.double().numpy()
        if not first:
            y = y * a
        got = ops.head_norm_gate(o.to(device), gate.to(device),
                                 w.to(device), 1e-6, group, ops.GATE_SILU,
                                 first, None, None, torch.float32)
        np.testing.assert_allclose(got.cpu().numpy(), y, atol=3e-5,
                                   rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_rmsnorm_pair_mean_and_ssm_gates(device):
    g = torch.Generator().manual_seed(8)
    a, b = torch.randn(6, 50, generator=g) * 4, torch.randn(6, 50,
                                                            generator=g)
    wa, wb = torch.randn(50, generator=g), torch.randn(50, generator=g)
    ref = 0.5 * (oracle.rms_unit(a.double().numpy(), 1e-5)
                 * wa.double().numpy()
                 + oracle.rms_unit(b.double().numpy(), 1e-5)
                 * wb.double().numpy())
    got = ops.rmsnorm_pair_mean(a.to(device), b.to(device), wa.to(device),
                                wb.to(device), 1e-5)
    np.testing.assert_allclose(got.cpu().numpy(), ref, atol=2e-5, rtol=2e-5)
    x = torch.tensor([[-30.0, -1.0, 0.0], [2.0, 30.0, 90.0]])
    al = torch.tensor([0.3, -1.0, 0.5])
    dt = oracle.softplus(x.double().numpy())
    decay, step = ops.ssm_gates(x.to(device), al.to(device))
    np.testing.assert_allclose(step.cpu().numpy(), dt, rtol=1e-5, atol=1e-12)
    np.testing.assert_allclose(
        decay.cpu().numpy(), np.exp(-np.exp(al.double().numpy()) * dt),
        rtol=1e-5, atol=1e-12)


def _attention_case(device, dtype, H, G, N, P, bs, ctx, scale, cap, coef,
                    every, boost=None):
    """Keys and values of one sequence of `ctx` tokens in scattered
    pages; every position is a query row.  boost = (query, key, factor)
    scales one query and one key so that a single score stands out."""
    g = torch.Generator().manual_seed(ctx + N)
    q = torch.randn(ctx, H, N, generator=g)
    k = torch.randn(ctx, G, N, generator=g)
    v = torch.randn(ctx, G, P, generator=g)
    if boost:
        qi, kj, f = boost
        k[kj] *= f
        q[qi] = k[kj].repeat_interleave(H // G, 0) * (1.0 / f)
    q, k, v = (x.to(dtype).float() for x in (q, k, v))
    ref = oracle.softcap_attention(q.double().numpy(), k.double().numpy(),
                                   v.double().numpy(), H, G, scale, cap,
                                   coef, every)
    nb = (ctx + bs - 1) // bs
    perm = torch.randperm(nb + 3, generator=g)[:nb].tolist()
    kc = torch.zeros(nb + 3, G, bs, N, dtype=dtype, device=device)
    vc = torch.zeros(nb + 3, G, bs, P, dtype=dtype, device=device)
    slots = [perm[j // bs] * bs + j % bs for j in range(ctx)]
    ops.append_paged_kv(k.reshape(ctx, -1).to(dtype).to(device),
                        v.reshape(ctx, -1).to(dtype).to(device), kc, vc,
                        i32(slots, device))
    out = ops.softcap_attention(
        q.reshape(ctx, -1).to(dtype).to(device), kc, vc,
        i32([perm], device), i32([0] * ctx, device),
        i32(list(range(ctx)), device), scale, cap, coef, every, 0, ctx,
        [ctx], i32([0, ctx], device), i32([0], device))
    return out.float().cpu().numpy().reshape(ctx, H, P), ref


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(4, 2, 6, 9, 4), (1, 1, 5, 3, 2),
                                  (6, 1, 20, 66, 8), (2, 2, 64, 64, 16)])
def test_softcap_attention_alone(device, dims):
    H, G, N, P, bs = dims
    out, ref = _attention_case(device, torch.float32, H, G, N, P, bs, 75,
                               0.4, 3.0, 0.5, 8)
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_attention_far_key_among_hundreds(device):
    """Query 299 matches key 3 only (boosted pair): its output must be
    that key's value, through every page border in between, and the cap
    must hold the score at softcap rather than letting it run away."""
    out, ref = _attention_case(device, torch.float32, 2, 1, 8, 5, 16, 300,
                               1.0, 12.0, 0.0, 1, boost=(299, 3, 6.0))
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)
    # the capped score 12 stands ~exp(12 - few) above the rest
    assert np.abs(out[299] - ref[299]).max() < 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_attention_query_stretch_steps(device):
    """The stretch changes exactly where floor((p + 1) / every) does."""
    out, ref = _attention_case(device, torch.float32, 2, 2, 4, 4, 4, 40,
                               0.9, 50.0, 2.0, 5)
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)
    base, _ = _attention_case(device, torch.float32, 2, 2, 4, 4, 4, 40, 0.9,
                              50.0, 0.0, 5)
    same = np.abs(out - base).reshape(40, -1).max(1) < 1e-6
    assert same[:4].all() and not same[4:].any()   # p + 1 >= 5 from row 4


@pytest.mark.gpu
@pytest.mark.parametrize("dims", [
    # H, G, N, P, page
    (4, 2, 64, 64, 16), (9, 3, 88, 176, 16), (8, 2, 128, 128, 8),
    (3, 1, 24, 72, 4), (2, 2, 40, 136, 16), (16, 1, 128, 64, 16)])
def test_attention_tile_kernel_bf16(dims):
    """The MFMA path over its padded instantiations: whole prompts
    (several tiles, a ragged last one), then a mixed launch of a prompt
    portion that continues a sequence beside decoded rows of others."""
    H, G, N, P, bs = dims
    dev = "cuda:0"
    out, ref = _attention_case(dev, torch.bfloat16, H, G, N, P, bs, 150,
                               N ** -0.5, 6.0, 0.4, 32)
    assert np.abs(out - ref).max() < 0.06
    out, ref = _attention_case(dev, torch.bfloat16, H, G, N, P, bs, 70,
                               1.0, 9.0, 0.0, 1, boost=(69, 2, 4.0))
    assert np.abs(out - ref).max() < 0.06
    # three sequences of 90, 130 and 64 cached tokens: the first brings
    # its last 37 rows as a portion, the others one decoded row each
    g = torch.Generator().manual_seed(N + P)
    lens, news = [90, 130, 64], [37, 1, 1]
    qs, refs, slots, tables = [], [], [], []
    nb = sum((L + bs - 1) // bs for L in lens)
    kc = torch.zeros(nb + 2, G, bs, N, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros(nb + 2, G, bs, P, dtype=torch.bfloat16, device=dev)
    perm = torch.randperm(nb + 2, generator=g).tolist()
    maxb = max((L + bs - 1) // bs for L in lens)
    for L, n in zip(lens, news):
        q = torch.randn(L, H, N, generator=g).bfloat16().float()
        k = torch.randn(L, G, N, generator=g).bfloat16().float()
        v = torch.randn(L, G, P, generator=g).bfloat16().float()
        r = oracle.softcap_attention(
            q.double().numpy(), k.double().numpy(), v.double().numpy(), H,
            G, N ** -0.5, 6.0, 0.4, 32)
        mine = [perm.pop() for _ in range((L + bs - 1) // bs)]
        tables.append(mine + [0] * (maxb - len(mine)))
        sl = [mine[j // bs] * bs + j % bs for j in range(L)]
        ops.append_paged_kv(k.reshape(L, -1).bfloat16().to(dev),
                            v.reshape(L, -1).bfloat16().to(dev), kc, vc,
                            i32(sl, dev))
        qs.append(q[L - n:].reshape(n, -1))
        refs.append(r[L - n:])
    cu = [0, 37, 38, 39]
    out = ops.softcap_attention(
        torch.cat(qs).bfloat16().to(dev), kc, vc, i32(tables, dev),
        i32([0] * 37 + [1, 2], dev),
        i32(list(range(53, 90)) + [129, 63], dev), N ** -0.5, 6.0, 0.4, 32,
        0, 37, [37], i32(cu, dev), i32([53, 129, 63], dev))
    got = out.float().cpu().numpy().reshape(39, H, P)
    assert np.abs(got - np.concatenate(refs)).max() < 0.06


# ---------------------------------------------------------------------------
# the engine against the oracle
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_layers_and_logits(tmp_path, device, name):
    cfg = CONFIGS[name]()
    W = oracle.random_weights(cfg, 11)
    eng = make_engine(tmp_path, cfg, W, device)
    t = toks(41, cfg["vocab"], 12)
    ref, taps_ref = oracle.forward(W, cfg, t)
    taps = []
    eng.model.tap = lambda i, x: taps.append(x.double().cpu().numpy())
    got = replay_all(eng, t, [41])
    eng.model.tap = None
    for i, (a, b) in enumerate(zip(taps, taps_ref)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), i
    close(got, ref, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_and_token_by_token(tmp_path, device, name):
    """The same request whole, token by token, and in ragged portions
    down to two tokens (cut inside pages and inside the filters' reach);
    pages and slots are reused from run to run."""
    cfg = CONFIGS[name]()
    W = oracle.random_weights(cfg, 13)
    eng = make_engine(tmp_path, cfg, W, device, blocks=16)
    t = toks(37, cfg["vocab"], 14)
    ref, _ = oracle.forward(W, cfg, t)
    for cuts in ([37], [1] * 37, [2, 2, 5, 1, 1, 9, 2, 3, 12],
                 [30] + [1] * 7, [3, 1, 33]):
        close(replay_all(eng, t, cuts), ref, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_against_each_alone(tmp_path, device):
    """Four unequal requests interleaved (portions beside single
    tokens, a request left out of steps, a fifth admitted into a freed
    slot and freed pages) give what each gives alone."""
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 15)
    eng = make_engine(tmp_path, cfg, W, device, blocks=36, slots=4)
    reqs = {n: toks(L, cfg["vocab"], 20 + i) for i, (n, L) in enumerate(
        [("a", 50), ("b", 23), ("c", 9), ("d", 31), ("e", 17)])}
    ref = {n: oracle.forward(W, cfg, t)[0] for n, t in reqs.items()}
    plan = [
        {"a": 3, "b": 3},
        {"a": 20, "c": 2},
        {"a": 1, "b": 17, "c": 1, "d": 2},
        {"a": 2, "c": 6, "d": 16},
        {"b": 1, "d": 1},
        {"a": 1, "b": 1, "d": 1},
        {"a": 13, "b": 1, "d": 11, "e": 5},     # e takes c's slot
        {"a": 10, "e": 1},
        {"e": 11},
    ]
    ids, at, got = {}, {n: 0 for n in reqs}, {n: [] for n in reqs}
    for step in plan:
        feeds, want = [], {}
        for n, k in step.items():
            if n not in ids:
                ids[n] = eng.open_stream()
            part = reqs[n][at[n]:at[n] + k]
            feeds.append((ids[n], part))
            want[ids[n]] = list(range(k))
            at[n] += k
        out = eng.replay_step(feeds, want)
        r = 0
        for n, k in step.items():
            got[n].append(out[r:r + k])
            r += k
        for n in list(step):
            if at[n] == len(reqs[n]):
                eng.close_stream(ids[n])
    for n in reqs:
        assert at[n] == len(reqs[n])
        close(torch.cat(got[n]), ref[n], 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(tmp_path, device):
    cfg = cfg_ones()
    W = oracle.random_weights(cfg, 16)
    eng = make_engine(tmp_path, cfg, W, device, blocks=80)
    t = toks(260, cfg["vocab"], 17)
    ref, _ = oracle.forward(W, cfg, t)
    close(replay_all(eng, t, [6] + [1] * 254), ref, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_mode(tmp_path, device):
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 18)
    eng = make_engine(tmp_path, cfg, W, device, dtype="bfloat16")
    t = toks(33, cfg["vocab"], 19)
    ref, _ = oracle.forward(W, cfg, t)
    whole = replay_all(eng, t, [33])
    close(whole, ref, 1e-1)
    close(replay_all(eng, t, [5, 2, 1, 1, 20, 4]), ref, 1e-1)


def _greedy(cfg, W, prompt, n):
    t = list(prompt)
    for _ in range(n):
        t.append(int(np.argmax(oracle.forward(W, cfg, t)[0][-1])))
    return t[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode", ["plain", "chunked_mixed"])
def test_greedy_generation_through_scheduler(tmp_path, device, mode):
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 21)
    kw = {}
    if mode == "chunked_mixed":
        kw = dict(enable_chunked_prefill=True, enable_mixed_batches=True,
                  max_batched_tokens=7)
    eng = make_engine(tmp_path, cfg, W, device, **kw)
    prompts = [toks(n, cfg["vocab"], 30 + n) for n in (5, 19, 11)]
    rids = [eng.add_request(p, SamplingParams(max_new_tokens=6,
                                              temperature=0.0))
            for p in prompts]
    for _ in range(200):
        if eng.is_finished():
            break
        eng.step()
    for rid, p in zip(rids, prompts):
        assert eng.get_output(rid).token_ids == _greedy(cfg, W, p, 6)


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_restarts_every_state(tmp_path, device):
    """A pool too small for both requests: the newer one is preempted,
    its slot buffers dropped with its pages, and it resumes by re-running
    its folded prompt from position 0."""
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 26)
    prompts = [toks(7, cfg["vocab"], 41), toks(6, cfg["vocab"], 42)]
    refs = [_greedy(cfg, W, p, 10) for p in prompts]
    eng = make_engine(tmp_path, cfg, W, device, blocks=8, block=4)
    sp = SamplingParams(max_new_tokens=10, temperature=0.0)
    ids = [eng.add_request(p, sp) for p in prompts]
    for _ in range(300):
        if eng.is_finished():
            break
        eng.step()
    assert eng.scheduler.num_preemptions > 0
    for i, r in zip(ids, refs):
        assert eng.get_output(i).token_ids == r


@pytest.mark.parametrize("device", DEVICES)
def test_forked_group_copies_every_slot_buffer(tmp_path, device):
    """n=2 from one prefill: the branch shares the prompt's pages and
    starts from a COPY of the parent's memories, filter histories,
    previous row and previous token."""
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 27)
    prompt = toks(10, cfg["vocab"], 43)     # 2 full pages + a partial one
    ref = _greedy(cfg, W, prompt, 5)
    eng = make_engine(tmp_path, cfg, W, device, blocks=32)
    ids = eng.add_request_group(
        prompt, SamplingParams(max_new_tokens=5, temperature=0.0), n=2)
    while not eng.is_finished():
        eng.step()
    assert eng.num_forks == 1
    for i in ids:
        assert eng.get_output(i).token_ids == ref


def test_table_sizes_from_tensors(tmp_path):
    """A config.json that leaves out the table sizes takes them from
    the checkpoint header."""
    cfg = cfg_ones()
    W = oracle.random_weights(cfg, 28)
    lean = {k: v for k, v in cfg.items() if k != "max_positions"}
    lean["embedding"] = {"scale": cfg["embedding"]["scale"],
                         "bigram": {"mul_prev": 1, "mul_cur": 1}}
    path = oracle.save_checkpoint(tmp_path / "m", lean, W)
    mc = model_config_from_dir(path)
    assert mc.max_position == cfg["max_positions"]
    assert mc.pair_hash.buckets == cfg["embedding"]["bigram"]["buckets"]


def test_registry_config_and_loader_errors(tmp_path):
    cfg = cfg_wide()
    W = oracle.random_weights(cfg, 22)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    mc = model_config_from_dir(path)
    assert isinstance(mc, FeditarConfig) and is_recurrent(mc)
    assert [l.type for l in mc.layers] == ["mamba2", "mlstm", "parallel"]
    assert mc.layers[2].mixer.right.decay_rank == 4
    assert mc.layers[0].mixer.conv_channels == 6 * 11 + 2 * 3 * 17
    assert mc.pair_hash.buckets == 53 and mc.max_position == 700
    with pytest.raises(ValueError, match="prefix caching"):
        LLMEngine(EngineConfig(model=mc, num_gpu_blocks=8, max_num_seqs=2,
                               enable_prefix_caching=True), device="cpu")
    bad = dict(W)
    bad["l0.mix.in"] = bad["l0.mix.in"][:-1]
    p2 = oracle.save_checkpoint(tmp_path / "bad", cfg, bad)
    with pytest.raises(ValueError, match="l0.mix.in"):
        make_engine(tmp_path / "e", cfg, bad, "cpu")
    del p2
    unknown = oracle.make_config(8, 9, [{"type": "lstm", "mixer": {},
                                         "mlp": None}])
    with pytest.raises(ValueError, match="unknown mixer"):
        FeditarConfig.from_dict(unknown)


def test_preset_runs_and_forks_copy_state(tmp_path):
    eng = LLMEngine(EngineConfig.tiny_feditar(), device="cpu")
    rid = eng.add_request(list(range(1, 20)),
                          SamplingParams(max_new_tokens=4, temperature=0.0))
    while not eng.is_finished():
        eng.step()
    assert len(eng.get_output(rid).token_ids) == 4
    # every slot buffer of every layer follows a fork
    caches = eng.kv_caches
    leaves = [t for t, kind in caches._all() if kind in ("state",
                                                         "slot_i32")]
    assert len(leaves) >= 2 * len(eng.model.layers)
    for t in leaves:
        t[1] = 3
    caches.copy_slot(1, 2)
    assert all(bool((t[2] == 3).all()) for t in leaves)


def test_local_provider_serves_a_checkpoint_directory(tmp_path):
    """The gateway's local provider with LOCAL_MODEL=hf picks the
    architecture from the directory's config.json and generates through
    the async engine with sampling."""
    import asyncio

    from inference_gateway_amd.config import LocalConfig
    from inference_gateway_amd.providers.local import LocalProvider

    cfg = oracle.make_config(48, 300, [
        oracle.mlstm_layer(2, 8, 6),
        oracle.parallel_layer(2, 1, 8, 10, 3, 0.2, 16, 0.35, 9.0, 3, 4,
                              ff=32)], max_positions=160)
    W = oracle.random_weights(cfg, 35)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    lc = LocalConfig(enabled=True, model="hf", max_num_seqs=4,
                     max_model_len=128)
    lc.num_gpu_blocks = 64
    lc.weights_path = path
    provider = LocalProvider(lc, device="cpu")
    try:
        assert isinstance(provider.engine.engine.cfg.model, FeditarConfig)

        async def go(temp):
            return await provider.chat_completions({
                "model": "local/hf",
                "messages": [{"role": "user", "content": "hi"}],
                "max_tokens": 3, "temperature": temp, "top_p": 0.9})

        assert asyncio.run(go(0))["usage"]["completion_tokens"] == 3
        assert asyncio.run(go(0.8))["usage"]["completion_tokens"] == 3
    finally:
        provider.engine.shutdown()


def test_trace_command(tmp_path):
    """bin/trace_run end to end on a small checkpoint: portions, a
    decoded token, a step with nothing wanted, a second request that
    reuses the first one's slot."""
    import json

    cfg = cfg_ones()
    W = oracle.random_weights(cfg, 23)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    a, b = toks(9, cfg["vocab"], 24), toks(4, cfg["vocab"], 25)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:5],
                                 "want": [0, 4]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[5:8], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [0]},
                                {"id": "b", "tokens": b, "want": [3]}],
         "end": ["a", "b"]},
    ]
    root = Path(__file__).resolve().parent.parent
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    r = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", path,
         "--dtype", "float32", "--out", str(tmp_path / "o"),
         "--max-tokens", "128"],
        input="".join(json.dumps(s) + "\n" for s in steps), text=True,
        capture_output=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [
        "done 0", "done 1", "done 2"]
    ra, rb = oracle.forward(W, cfg, a)[0], oracle.forward(W, cfg, b)[0]
    V = cfg["vocab"]
    g0 = np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(-1, V)
    g2 = np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(-1, V)
    assert not (tmp_path / "o" / "1.f32").exists()
    close(g0, ra[[0, 4]], 2e-4)
    close(g2, np.stack([ra[8], rb[3]]), 2e-4)
