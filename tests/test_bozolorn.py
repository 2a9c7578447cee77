"""Bozolorn (sandwich-norm decoder: chunked distance-biased attention /
parallel sink attention + gated delta rule, group-routed experts, token
side input) against a plain float64 model written from the equations
(tests/bozolorn_oracle.py).

Every test builds its own small configuration and random checkpoint; the
engine reads it through the product loader.  Device-parametrized: the CPU
cases run the reference ops, the GPU cases the HIP kernels, both through
the same engine, cache manager and scheduler.
"""
import json
import math
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import bozolorn_oracle as oracle
from inference_gateway_amd import ops
from inference_gateway_amd.engine.config import (BozolornConfig,
                                                 EngineConfig,
                                                 SamplingParams,
                                                 YarnRotarySpec)
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


# configurations; sizes all differ from one another
def cfg_small():
    moe = oracle.moe_ff(6, 2, 3, 2, 12, 1.5)
    return oracle.make_config(40, 61, [
        oracle.parallel_layer(4, 2, 6, 9, 0.3,
                              oracle.rot(4, 100.0, 3.0, 16, 4.0, 1.0),
                              4, 2, 5, 7, 3, mlp=moe),
        oracle.attention_layer(4, 2, 6, 5, 7, 0.4, mlp=moe),
        oracle.parallel_layer(2, 1, 8, 4, 0.25, oracle.rot(8, 50.0),
                              2, 2, 6, 6, 2),
        oracle.attention_layer(4, 2, 6, 5, 5, 0.3, mlp=moe, kv_from=1)],
        side=3)


def cfg_ones():
    """Single heads and groups, one expert group, one chosen expert, a
    one-tap filter, a chunk of one page, no rotation on one layer, no
    token side input, an attention layer first."""
    return oracle.make_config(24, 37, [
        oracle.attention_layer(1, 1, 5, 3, 4, 0.45,
                               mlp=oracle.moe_ff(3, 1, 1, 1, 8, 0.8)),
        oracle.parallel_layer(1, 1, 4, 3, 0.5, None, 1, 1, 3, 5, 1),
        oracle.parallel_layer(3, 3, 4, 4, 0.5,
                              oracle.rot(2, 10.0, 2.0, 8, 2.0, 0.5),
                              3, 1, 4, 2, 5,
                              mlp=oracle.moe_ff(4, 2, 4, 2, 6, 30.0)),
        oracle.attention_layer(2, 1, 3, 4, 1000, 0.6)],
        scale=1.0, eps=1e-6)


def cfg_wide():
    """Widths that straddle the kernels' tile sizes: more than 64 value
    entries per head, key widths off the powers of two, many heads on
    one key/value head, groups of one expert."""
    return oracle.make_config(72, 83, [
        oracle.parallel_layer(6, 1, 20, 66, 0.22,
                              oracle.rot(12, 1000.0, 8.0, 32, 16.0, 2.0),
                              4, 2, 33, 70, 4,
                              mlp=oracle.moe_ff(5, 3, 5, 4, 10, 2.5)),
        oracle.attention_layer(6, 3, 24, 72, 33, 0.2),
        oracle.attention_layer(6, 3, 24, 72, 16, 0.25, kv_from=1,
                               mlp=oracle.moe_ff(8, 3, 2, 1, 9, 1.0))],
        side=5)


CONFIGS = {"small": cfg_small, "ones": cfg_ones, "wide": cfg_wide}


def make_engine(tmp_path, cfg, W, device, dtype="float32", blocks=48,
                block=4, slots=4, **kw):
    path = oracle.save_checkpoint(Path(tmp_path) / "ckpt", cfg, W)
    ecfg = EngineConfig(
        model=model_config_from_dir(path), block_size=block,
        num_gpu_blocks=blocks, max_num_seqs=slots,
        max_batched_tokens=kw.pop("max_batched_tokens", 4096),
        max_model_len=1024, use_hip_graphs=False,
        weights_path=path, dtype=dtype, **kw)
    return LLMEngine(ecfg, device=_dev(device))


def close(got, ref, tol, most=1.0):
    """Mean-free relative RMS difference per row, like a logit check.
    most < 1: that share of the rows must pass (bfloat16 rounding can
    flip a close expert choice, which moves a whole row)."""
    got = torch.as_tensor(np.asarray(got.cpu() if torch.is_tensor(got)
                                     else got)).double()
    ref = torch.as_tensor(np.asarray(ref)).double()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()
    if most < 1.0:
        err = err.sort().values[:max(1, int(most * err.numel()))]
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
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(2, 1, 5, 7), (3, 3, 16, 64),
                                  (4, 2, 40, 70), (1, 1, 1, 1)])
def test_delta_scan_two_steps(device, dims):
    """A fresh sequence over a stale slot, a continued one and a one-row
    one, in two steps, against the recurrence written out; q and k are
    normalised inside."""
    H, G, N, P = dims
    g = torch.Generator().manual_seed(N + P)
    lens = [21, 9, 1]
    seqs = []
    for L in lens:
        q, k = torch.randn(L, G, N, generator=g), torch.randn(L, G, N,
                                                             generator=g)
        v = torch.randn(L, H, P, generator=g)
        a = torch.rand(L, H, generator=g) * 0.6 + 0.4
        b = torch.rand(L, H, generator=g)
        qn = q.double().numpy()
        kn = k.double().numpy()
        qn = qn / np.sqrt((qn * qn).sum(-1, keepdims=True) + 1e-6) * 0.3
        kn = kn / np.sqrt((kn * kn).sum(-1, keepdims=True) + 1e-6)
        ref = oracle.delta_rule(np.repeat(qn, H // G, 1),
                                np.repeat(kn, H // G, 1),
                                v.double().numpy(), b.double().numpy(),
                                a.double().numpy())
        seqs.append((q, k, v, a, b, ref))
    state = torch.randn(5, H * N * P, generator=g).to(device)   # stale
    slots = [3, 0, 4]
    for step, plan in enumerate([[(0, 17), (0, 2), (0, 1)],
                                 [(17, 4), (2, 7), None]]):
        rows, starts, sl, parts, want = [], [], [], [], []
        for s, pl in enumerate(plan):
            if pl is None:
                continue
            a0, n = pl
            rows.append(n), starts.append(a0), sl.append(slots[s])
            parts.append([x[a0:a0 + n] for x in seqs[s][:5]])
            want.append(seqs[s][5][a0:a0 + n])
        cu, st, so, _rs, _ = ragged(rows, starts, sl, device)
        q, k, v, a, b = (torch.cat([p[j] for p in parts]).to(device)
                         for j in range(5))
        out = ops.delta_scan(q, k, v, a.contiguous(), b.contiguous(), state,
                             cu, st, so, rows, 1e-6, 0.3)
        np.testing.assert_allclose(out.cpu().numpy(), np.concatenate(want),
                                   atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_overwrites_a_key(device):
    """With write strength 1 and no decay, writing a second value under
    the same unit key replaces the first: the read-out returns the new
    value, not the sum (what a plain outer-product memory would give)."""
    N, P = 8, 6
    k = torch.zeros(3, 1, N)
    k[:, 0, 2] = 5.0                         # same direction, any length
    v = torch.tensor([[[1.0] * P], [[-2.0] * P], [[0.5] * P]])
    ones = torch.ones(3, 1)
    state = torch.zeros(1, N * P, device=device)
    out = ops.delta_scan(k.to(device), k.to(device), v.to(device),
                         ones.to(device), ones.to(device), state,
                         i32([0, 3], device), i32([0], device),
                         i32([0], device), [3], 1e-6, 1.0)
    np.testing.assert_allclose(out.cpu().numpy(), v.numpy(), atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_decay_beta_gates(device):
    pre = torch.tensor([[-30.0, -1.0, 0.0, 3.0, -40.0, 0.2],
                        [2.0, 30.0, 90.0, -3.0, 40.0, 0.0]])
    al = torch.tensor([0.3, -1.0, 0.5])
    db = torch.tensor([0.1, -0.2, 1.5])
    decay, beta = ops.decay_beta_gates(pre.to(device), al.to(device),
                                       db.to(device))
    x = pre.double().numpy()
    dt = oracle.softplus(x[:, :3] + db.double().numpy())
    np.testing.assert_allclose(decay.cpu().numpy(),
                               np.exp(-np.exp(al.double().numpy()) * dt),
                               rtol=1e-5, atol=1e-12)
    np.testing.assert_allclose(beta.cpu().numpy(), oracle.sigmoid(x[:, 3:]),
                               rtol=1e-5, atol=1e-12)


def _route_ref(logits, corr, top, groups, keep):
    ids, ws = [], []
    for z in logits:
        i, w = oracle.route(z, corr, top, groups, keep)
        ids.append(sorted(i.tolist()))
        ws.append(dict(zip(i.tolist(), w.tolist())))
    return ids, ws


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("shape", [(8, 3, 4, 2), (6, 2, 1, 1), (5, 3, 5, 4),
                                   (64, 8, 8, 3), (12, 4, 3, 3),
                                   (9, 1, 3, 1)])
def test_group_route(device, shape):
    E, K, groups, keep = shape
    g = torch.Generator().manual_seed(E * K)
    logits = torch.randn(50, E, generator=g) * 2.0
    corr = torch.randn(E, generator=g) * 0.5 - 0.8    # negative choices
    w, idx, dst = ops.moe_group_route(logits.to(device), corr.to(device), K,
                                      groups, keep, 64)
    ids, ws = _route_ref(logits.double().numpy(), corr.double().numpy(), K,
                         groups, keep)
    idx, w = idx.cpu().tolist(), w.cpu().tolist()
    for t in range(50):
        assert sorted(idx[t]) == ids[t], t
        for e, x in zip(idx[t], w[t]):
            assert abs(x - ws[t][e]) < 1e-6
    if dst is not None:
        # padded-dispatch rows: inside the expert's segment, all distinct
        d = dst.cpu().tolist()
        assert len(set(d)) == len(d)
        flat = [e for row in idx for e in row]
        assert all(e * 64 <= r < e * 64 + 50 for e, r in zip(flat, d))


@pytest.mark.parametrize("device", DEVICES)
def test_group_route_masks_with_minus_infinity(device):
    """All choice scores negative: an expert of a dropped group must
    lose against every expert of a kept group (a dropped score counted
    as 0 would win), the correction moves the choice but not the weight,
    and a group scores by its best TWO experts, not its best one."""
    logits = torch.tensor([[3.0, -9.0, 2.0, 1.9, -8.0, -8.5]])
    corr = torch.tensor([-5.0] * 6)
    # group sums: {0,1}: s0+s1-10, {2,3}: s2+s3-10 (largest), {4,5}: tiny
    w, idx, _ = ops.moe_group_route(logits.to(device), corr.to(device), 2, 3,
                                    1, 0)
    assert sorted(idx[0].tolist()) == [2, 3]
    np.testing.assert_allclose(
        sorted(w[0].tolist()),
        sorted(oracle.sigmoid(np.array([2.0, 1.9])).tolist()), rtol=1e-6)
    # a correction lifts expert 5 into the choice; its weight stays s_5
    corr2 = torch.tensor([0.0, 0.0, 0.0, 0.0, 3.0, 3.0])
    w, idx, _ = ops.moe_group_route(logits.to(device), corr2.to(device), 1,
                                    3, 1, 0)
    assert idx[0].tolist() == [4]
    assert abs(float(w[0, 0]) - oracle.sigmoid(-8.0)) < 1e-7


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D", [50, 256, 700])
def test_add_normed_rmsnorm(device, D):
    g = torch.Generator().manual_seed(D)
    res = torch.randn(5, D, generator=g) * 3
    delta = torch.randn(5, D + 4, generator=g) * 7
    wp, wn = torch.randn(D, generator=g), torch.randn(D, generator=g)
    r = res.double().numpy()
    r1 = r + oracle.rms_unit(delta[:, :D].double().numpy(), 1e-5) \
        * wp.double().numpy()
    x = res.clone().to(device)
    out = ops.add_normed_rmsnorm(x, delta.to(device)[:, :D], wp.to(device),
                                 wn.to(device), 1e-5, torch.float32)
    np.testing.assert_allclose(x.cpu().numpy(), r1, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(
        out.cpu().numpy(), oracle.rms_unit(r1, 1e-5) * wn.double().numpy(),
        atol=2e-5, rtol=2e-5)
    # nothing to add; no outgoing norm
    x = res.clone().to(device)
    out = ops.add_normed_rmsnorm(x, None, None, wn.to(device), 1e-5,
                                 torch.float32)
    np.testing.assert_allclose(
        out.cpu().numpy(), oracle.rms_unit(r, 1e-5) * wn.double().numpy(),
        atol=2e-5, rtol=2e-5)
    out = ops.add_normed_rmsnorm(x, delta.to(device)[:, :D].bfloat16(),
                                 wp.to(device), None, 1e-5, torch.bfloat16)
    assert out.dtype == torch.bfloat16
    np.testing.assert_allclose(out.float().cpu().numpy(), x.cpu().numpy(),
                               rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("device", DEVICES)
def test_gelu_mul_rows(device):
    g = torch.Generator().manual_seed(3)
    z = torch.randn(7, 5, generator=g) * 3
    table = torch.randn(11, 23, generator=g)
    tok = torch.tensor([3, 0, 10, 3, 7, 1, 9])
    out = ops.gelu_mul_rows(z.to(device), table.to(device), tok.to(device),
                            10)
    ref = oracle.gelu_tanh(z.double().numpy()) \
        * table.double().numpy()[tok.numpy(), 10:15]
    np.testing.assert_allclose(out.cpu().numpy(), ref, atol=2e-6, rtol=2e-5)


def test_yarn_frequencies_against_the_formula():
    spec = YarnRotarySpec(base=500.0, dims=12, factor=4.0, original=40.0,
                          fast=8.0, slow=0.5)
    f, mag = spec.frequencies()
    rf, rmag = oracle.rotary_frequencies(
        {"dims": 12, "base": 500.0,
         "scaling": {"factor": 4.0, "original": 40.0, "fast": 8.0,
                     "slow": 0.5}})
    np.testing.assert_allclose(f, rf, rtol=1e-12)
    assert abs(mag - rmag) < 1e-12
    # pair 0 keeps its frequency, the last pair is slowed by the factor,
    # something in between is interpolated
    plain = [500.0 ** (-2.0 * i / 12) for i in range(6)]
    assert f[0] == plain[0] and abs(f[5] - plain[5] / 4.0) < 1e-15
    assert any(plain[i] / 4.0 < f[i] < plain[i] for i in range(1, 5))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(4, 2, 6, 9, 4), (1, 1, 5, 3, 0),
                                  (3, 3, 24, 16, 16), (2, 1, 7, 5, 6)])
def test_qk_norm_rope_append(device, dims):
    """Per-head norm with a shared weight, rotation of only the first
    entries (scaled cos/sin), keys and values into scattered pages."""
    H, G, N, P, rd = dims
    T, bs = 13, 4
    g = torch.Generator().manual_seed(N)
    proj = torch.randn(T, (H + G) * N + G * P + 5, generator=g)
    qw, kw = torch.randn(N, generator=g), torch.randn(N, generator=g)
    rot = {"dims": rd, "base": 30.0,
           "scaling": {"factor": 2.0, "original": 16, "fast": 4.0,
                       "slow": 1.0}} if rd else None
    pos = [40, 41, 42, 0, 1, 2, 3, 4, 5, 6, 7, 8, 900]
    x = proj.double().numpy()

    def expect(block, heads, w):
        y = oracle.rms_unit(block.reshape(T, heads, N), 1e-5) \
            * w.double().numpy()
        if not rot:
            return y
        out = np.empty_like(y)
        for t, p in enumerate(pos):        # the oracle rotates by index
            big = np.zeros((p + 1, heads, N))
            big[p] = y[t]
            out[t] = oracle.rotate_pairs(big, rot)[p]
        return out

    q_ref = expect(x[:, :H * N], H, qw)
    k_ref = expect(x[:, H * N:(H + G) * N], G, kw)
    inv, mag = (None, 1.0)
    if rot:
        fr, mag = oracle.rotary_frequencies(rot)
        inv = f32(fr, device)
    kc = torch.zeros(9, G, bs, N, device=device)
    vc = torch.zeros(9, G, bs, P, device=device)
    slots = [7 * bs + 1, 7 * bs + 2, 2 * bs + 3] + list(range(3 * bs,
                                                              3 * bs + 10))
    q = ops.qk_norm_rope_append(
        proj.to(device), i32(pos, device), i32(slots, device), kc, vc,
        qw.to(device), kw.to(device), inv, mag, 1e-5, H, G, N, P)
    np.testing.assert_allclose(q.cpu().numpy().reshape(T, H, N), q_ref,
                               atol=3e-5, rtol=3e-5)
    for t, s in enumerate(slots):
        np.testing.assert_allclose(kc[s // bs, :, s % bs].cpu().numpy(),
                                   k_ref[t], atol=3e-5, rtol=3e-5)
        np.testing.assert_allclose(
            vc[s // bs, :, s % bs].cpu().numpy().reshape(-1),
            x[t, (H + G) * N:(H + G) * N + G * P], atol=1e-6)


def _attention_case(device, dtype, H, G, N, P, bs, ctx, scale, kind, chunk=0,
                    boost=None, gate=False):
    """Keys and values of one sequence of `ctx` tokens in scattered
    pages; every position is a query row.  kind = "bias" (distance
    slopes inside position chunks) or "sink".  boost = (query, key,
    factor) scales one query and one key so that a single score stands
    out."""
    g = torch.Generator().manual_seed(ctx + N)
    q = torch.randn(ctx, H, N, generator=g)
    k = torch.randn(ctx, G, N, generator=g)
    v = torch.randn(ctx, G, P, generator=g)
    gt = torch.randn(ctx, H * P + 3, generator=g)
    if boost:
        qi, kj, f = boost
        k[kj] *= f
        q[qi] = k[kj].repeat_interleave(H // G, 0) * (1.0 / f)
    q, k, v, gt = (x.to(dtype).float() for x in (q, k, v, gt))
    qn, kn, vn = (x.double().numpy() for x in (q, k, v))
    if kind == "bias":
        ref = oracle.chunk_bias_attention(qn, kn, vn, H, G, scale, chunk)
        extra = dict(slopes=f32(oracle.distance_slopes(H), device),
                     chunk=chunk)
    else:
        ref = oracle.sink_attention(qn, kn, vn, H, G, scale)
        extra = dict(sinks=torch.zeros(H, device=device))
    if gate:
        ref = ref * oracle.sigmoid(
            gt[:, :H * P].double().numpy()).reshape(ctx, H, P)
        extra["gate"] = gt.to(dtype).to(device)[:, :H * P]
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
        i32(list(range(ctx)), device), scale, 0.0, 0.0, 1, 0, ctx,
        [ctx], i32([0, ctx], device), i32([0], device), **extra)
    return out.float().cpu().numpy().reshape(ctx, H, P), ref


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(4, 2, 6, 9, 4, 7), (1, 1, 5, 3, 2, 1),
                                  (6, 1, 20, 66, 8, 30),
                                  (2, 2, 64, 64, 16, 64),
                                  (8, 4, 16, 8, 4, 0)])
def test_chunk_bias_attention_alone(device, dims):
    H, G, N, P, bs, chunk = dims
    out, ref = _attention_case(device, torch.float32, H, G, N, P, bs, 75,
                               0.4, "bias", chunk, gate=True)
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dims", [(4, 2, 6, 9, 4), (1, 1, 5, 3, 2),
                                  (6, 1, 20, 66, 8), (2, 2, 64, 64, 16)])
def test_sink_attention_alone(device, dims):
    H, G, N, P, bs = dims
    out, ref = _attention_case(device, torch.float32, H, G, N, P, bs, 75,
                               0.4, "sink")
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_weight_when_every_score_is_low(device):
    """Scores far below zero: the sink owns the denominator and the
    output shrinks to almost nothing; a softmax without it would return
    an average of the values."""
    g = torch.Generator().manual_seed(5)
    ctx, N, P = 20, 4, 3
    q = torch.ones(ctx, 1, N)
    k = -torch.ones(ctx, 1, N) * 3.0          # every score = -12
    v = torch.randn(ctx, 1, P, generator=g) + 2.0
    kc = torch.zeros(6, 1, 4, N, device=device)
    vc = torch.zeros(6, 1, 4, P, device=device)
    ops.append_paged_kv(k.reshape(ctx, -1).to(device),
                        v.reshape(ctx, -1).to(device), kc, vc,
                        i32(list(range(4, 4 + ctx)), device))
    table = i32([[1, 2, 3, 4, 5]], device)
    args = (q.reshape(ctx, -1).to(device), kc, vc, table,
            i32([0] * ctx, device), i32(list(range(ctx)), device), 1.0, 0.0,
            0.0, 1, 0, ctx, [ctx], i32([0, ctx], device), i32([0], device))
    with_sink = ops.softcap_attention(*args, sinks=torch.zeros(
        1, device=device))
    plain = ops.softcap_attention(*args)
    ref = oracle.sink_attention(q.double().numpy(), k.double().numpy(),
                                v.double().numpy(), 1, 1, 1.0)
    np.testing.assert_allclose(with_sink.cpu().numpy(), ref.reshape(ctx, P),
                               atol=1e-8, rtol=1e-4)
    assert float(with_sink.abs().max()) < 1e-3 < float(plain.abs().min())


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(device):
    """Query 299 matches key 3 only (boosted pair): with the sink
    attention its output must be that key's value through every page
    border in between; with the distance bias the same far key loses
    296 slopes of score, exactly as the formula says."""
    out, ref = _attention_case(device, torch.float32, 2, 1, 8, 5, 16, 300,
                               1.0, "sink", boost=(299, 3, 3.0))
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)
    out, ref = _attention_case(device, torch.float32, 2, 1, 8, 5, 16, 300,
                               1.0, "bias", 0, boost=(299, 3, 3.0))
    np.testing.assert_allclose(out, ref, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("chunk", [5, 16, 24])
def test_chunk_edges_in_prompt_and_decode(device, chunk):
    """One boosted key sits at the last position of a chunk.  The
    queries of that chunk see it; the first query of the next chunk
    does not (its output is its own value alone).  The same rows are
    then run as single decoded rows."""
    H, G, N, P, bs, ctx = 2, 1, 8, 4, 4, 3 * chunk + 2
    edge = 2 * chunk - 1
    g = torch.Generator().manual_seed(chunk)
    q = torch.randn(ctx, H, N, generator=g) * 0.1
    k = torch.randn(ctx, G, N, generator=g) * 0.1
    v = torch.randn(ctx, G, P, generator=g)
    k[edge] = 4.0
    q[edge] = q[edge + 1] = 4.0               # both would love that key
    ref = oracle.chunk_bias_attention(q.double().numpy(), k.double().numpy(),
                                      v.double().numpy(), H, G, 1.0, chunk)
    assert np.abs(ref[edge] - v[edge].numpy()).max() < 1e-3
    assert np.abs(ref[edge + 1] - v[edge + 1].numpy()).max() < 1e-12
    nb = (ctx + bs - 1) // bs
    kc = torch.zeros(nb + 1, G, bs, N, device=device)
    vc = torch.zeros(nb + 1, G, bs, P, device=device)
    ops.append_paged_kv(k.reshape(ctx, -1).to(device),
                        v.reshape(ctx, -1).to(device), kc, vc,
                        i32(list(range(bs, bs + ctx)), device))
    table = i32([list(range(1, nb + 1))], device)
    slopes = f32(oracle.distance_slopes(H), device)
    whole = ops.softcap_attention(
        q.reshape(ctx, -1).to(device), kc, vc, table, i32([0] * ctx, device),
        i32(list(range(ctx)), device), 1.0, 0.0, 0.0, 1, 0, ctx, [ctx],
        i32([0, ctx], device), i32([0], device), slopes=slopes, chunk=chunk)
    np.testing.assert_allclose(whole.cpu().numpy().reshape(ctx, H, P), ref,
                               atol=3e-5, rtol=3e-5)
    for p in (edge - 1, edge, edge + 1, edge + 2, ctx - 1):
        one = ops.softcap_attention(
            q[p].reshape(1, -1).to(device), kc, vc, table, i32([0], device),
            i32([p], device), 1.0, 0.0, 0.0, 1, 0, 0, None,
            i32([0, 1], device), i32([p], device), slopes=slopes,
            chunk=chunk)
        np.testing.assert_allclose(one.cpu().numpy().reshape(H, P), ref[p],
                                   atol=3e-5, rtol=3e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dims", [
    # H, G, N, P, page, chunk
    (4, 2, 64, 64, 16, 48), (9, 3, 88, 176, 16, 100), (8, 2, 128, 128, 8, 0),
    (3, 1, 24, 72, 4, 70), (16, 1, 128, 64, 16, 33)])
def test_attention_tile_kernel_bf16(dims):
    """The MFMA path with slopes + chunks + gate and with the sink over
    its padded instantiations: whole prompts (several tiles, a ragged
    last one, chunks that start inside a tile), then a mixed launch of a
    prompt portion that continues a sequence beside decoded rows."""
    H, G, N, P, bs, chunk = dims
    dev = "cuda:0"
    out, ref = _attention_case(dev, torch.bfloat16, H, G, N, P, bs, 150,
                               N ** -0.5, "bias", chunk, gate=True)
    assert np.abs(out - ref).max() < 0.06
    out, ref = _attention_case(dev, torch.bfloat16, H, G, N, P, bs, 150,
                               N ** -0.5, "sink")
    assert np.abs(out - ref).max() < 0.06
    out, ref = _attention_case(dev, torch.bfloat16, H, G, N, P, bs, 70,
                               1.0, "sink", boost=(69, 2, 2.0))
    assert np.abs(out - ref).max() < 0.06
    # three sequences of 90, 130 and 64 cached tokens: the first brings
    # its last 37 rows as a portion, the others one decoded row each
    g = torch.Generator().manual_seed(N + P)
    lens, news = [90, 130, 64], [37, 1, 1]
    for kind in ("bias", "sink"):
        qs, refs, tables = [], [], []
        nb = sum((L + bs - 1) // bs for L in lens)
        kc = torch.zeros(nb + 2, G, bs, N, dtype=torch.bfloat16, device=dev)
        vc = torch.zeros(nb + 2, G, bs, P, dtype=torch.bfloat16, device=dev)
        perm = torch.randperm(nb + 2, generator=g).tolist()
        maxb = max((L + bs - 1) // bs for L in lens)
        for L, n in zip(lens, news):
            q = torch.randn(L, H, N, generator=g).bfloat16().float()
            k = torch.randn(L, G, N, generator=g).bfloat16().float()
            v = torch.randn(L, G, P, generator=g).bfloat16().float()
            if kind == "bias":
                r = oracle.chunk_bias_attention(
                    q.double().numpy(), k.double().numpy(),
                    v.double().numpy(), H, G, N ** -0.5, chunk)
            else:
                r = oracle.sink_attention(
                    q.double().numpy(), k.double().numpy(),
                    v.double().numpy(), H, G, N ** -0.5)
            mine = [perm.pop() for _ in range((L + bs - 1) // bs)]
            tables.append(mine + [0] * (maxb - len(mine)))
            sl = [mine[j // bs] * bs + j % bs for j in range(L)]
            ops.append_paged_kv(k.reshape(L, -1).bfloat16().to(dev),
                                v.reshape(L, -1).bfloat16().to(dev), kc, vc,
                                i32(sl, dev))
            qs.append(q[L - n:].reshape(n, -1))
            refs.append(r[L - n:])
        extra = (dict(slopes=f32(oracle.distance_slopes(H), dev),
                      chunk=chunk) if kind == "bias"
                 else dict(sinks=torch.zeros(H, device=dev)))
        out = ops.softcap_attention(
            torch.cat(qs).bfloat16().to(dev), kc, vc, i32(tables, dev),
            i32([0] * 37 + [1, 2], dev),
            i32(list(range(53, 90)) + [129, 63], dev), N ** -0.5, 0.0, 0.0,
            1, 0, 37, [37], i32([0, 37, 38, 39], dev),
            i32([53, 129, 63], dev), **extra)
        got = out.float().cpu().numpy().reshape(39, H, P)
        assert np.abs(got - np.concatenate(refs)).max() < 0.06, kind


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
    assert len(taps) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(taps, taps_ref)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), i
    close(got, ref, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_and_token_by_token(tmp_path, device, name):
    """The same request whole, token by token, and in ragged portions
    down to two tokens (cut inside pages, chunks and the filters' reach);
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
def test_first_tokens_in_used_slots(tmp_path, device):
    """Requests of one, two and three tokens admitted into slots and
    pages that longer requests have just left: the filter sees zeros
    before position 0, the memory starts empty, the sink faces a single
    key; a one-token request beside portions of others."""
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 61)
    eng = make_engine(tmp_path, cfg, W, device, blocks=24, slots=3)
    for n in (19, 23, 11):                     # dirty every slot and page
        replay_all(eng, toks(n, cfg["vocab"], 60 + n), [n])
    reqs = [toks(n, cfg["vocab"], 70 + n) for n in (1, 2, 3)]
    refs = [oracle.forward(W, cfg, t)[0] for t in reqs]
    ids = [eng.open_stream() for _ in reqs]
    out = eng.replay_step(
        [(i, t[:2]) for i, t in zip(ids, reqs)],
        {i: list(range(min(2, len(t)))) for i, t in zip(ids, reqs)})
    close(out, np.concatenate([r[:2] for r in refs]), 2e-4)
    out = eng.replay_step([(ids[2], reqs[2][2:])], {ids[2]: [0]})
    close(out, refs[2][2:], 2e-4)
    for i in ids:
        eng.close_stream(i)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(tmp_path, device):
    cfg = cfg_ones()
    W = oracle.random_weights(cfg, 16)
    eng = make_engine(tmp_path, cfg, W, device, blocks=80)
    t = toks(260, cfg["vocab"], 17)
    ref, _ = oracle.forward(W, cfg, t)
    close(replay_all(eng, t, [6] + [1] * 254), ref, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_borrowed_keys_follow_the_source_layer(tmp_path, device):
    """The borrowing layer reads the pages its source layer wrote in the
    SAME step, also when the request arrives in portions; making the
    source's keys useless changes the borrower's output too."""
    cfg = cfg_wide()
    W = oracle.random_weights(cfg, 31)
    t = toks(45, cfg["vocab"], 32)
    eng = make_engine(tmp_path / "a", cfg, W, device)
    ref, _ = oracle.forward(W, cfg, t)
    close(replay_all(eng, t, [20, 1, 1, 23]), ref, 2e-4)
    W2 = dict(W)
    W2["l1.mix.k"] = W["l1.mix.k"] * 0.0
    ref2, taps2 = oracle.forward(W2, cfg, t)
    assert np.abs(ref2 - ref).max() > 1e-3
    eng2 = make_engine(tmp_path / "b", cfg, W2, device)
    close(replay_all(eng2, t, [45]), ref2, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_mode(tmp_path, device):
    cfg = cfg_small()
    W = oracle.random_weights(cfg, 18)
    eng = make_engine(tmp_path, cfg, W, device, dtype="bfloat16")
    t = toks(33, cfg["vocab"], 19)
    ref, _ = oracle.forward(W, cfg, t)
    whole = replay_all(eng, t, [33])
    close(whole, ref, 1e-1, most=0.85)
    close(replay_all(eng, t, [5, 2, 1, 1, 20, 4]), ref, 1e-1, most=0.85)


@pytest.mark.gpu
def test_bfloat16_tile_sizes_through_the_engine(tmp_path):
    """Head sizes that take the MFMA attention path (multiples of 8), a
    prompt of several tiles, portions and decoded rows, in bfloat16."""
    moe = oracle.moe_ff(8, 2, 4, 2, 32, 3.0)
    cfg = oracle.make_config(128, 97, [
        oracle.parallel_layer(4, 2, 32, 16, 0.18,
                              oracle.rot(16, 10000.0, 4.0, 64, 32.0, 1.0),
                              4, 2, 16, 32, 4, mlp=moe),
        oracle.attention_layer(4, 4, 16, 24, 50, 0.25, mlp=moe),
        oracle.attention_layer(4, 4, 16, 24, 90, 0.25, kv_from=1)], side=8)
    W = oracle.random_weights(cfg, 51)
    eng = make_engine(tmp_path, cfg, W, "cuda", dtype="bfloat16", blocks=40,
                      block=16)
    t = toks(200, cfg["vocab"], 52)
    ref, _ = oracle.forward(W, cfg, t)
    close(replay_all(eng, t, [200]), ref, 1e-1, most=0.85)
    close(replay_all(eng, t, [70, 2, 100, 1, 1, 26]), ref, 1e-1, most=0.85)


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
    starts from a COPY of the parent's memory and filter history."""
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


def test_registry_config_and_loader_errors(tmp_path):
    cfg = cfg_wide()
    W = oracle.random_weights(cfg, 22)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    mc = model_config_from_dir(path)
    assert isinstance(mc, BozolornConfig) and is_recurrent(mc)
    assert [l.type for l in mc.layers] == ["parallel", "attention",
                                           "attention"]
    assert mc.layers[2].mixer.kv_from == 1 and mc.layers[1].mixer.chunk == 33
    assert mc.layers[0].mixer.right.conv_channels == 2 * 2 * 33 + 4 * 70
    assert mc.layers[0].mlp.keep == 4 and mc.side_dim == 5
    assert mc.layers[0].mixer.left.rot.dims == 12
    # only the layers that own keys and values page anything
    assert mc.kv_bytes_per_token(2) == 2 * ((20 + 66) + 3 * (24 + 72))
    with pytest.raises(ValueError, match="prefix caching"):
        LLMEngine(EngineConfig(model=mc, num_gpu_blocks=8, max_num_seqs=2,
                               enable_prefix_caching=True), device="cpu")
    bad = dict(W)
    bad["l1.mix.k"] = bad["l1.mix.k"][:-1]
    with pytest.raises(ValueError, match="l1.mix.q"):
        make_engine(tmp_path / "e", cfg, bad, "cpu")
    unknown = oracle.make_config(8, 9, [{"type": "lstm", "mixer": {},
                                         "mlp": None}])
    with pytest.raises(ValueError, match="unknown mixer"):
        BozolornConfig.from_dict(unknown)
    forward = oracle.make_config(8, 9, [
        oracle.attention_layer(1, 1, 4, 4, 8, 0.5, kv_from=1),
        oracle.attention_layer(1, 1, 4, 4, 8, 0.5)])
    with pytest.raises(ValueError, match="kv_from"):
        BozolornConfig.from_dict(forward)
    # attention-only models keep no per-slot state
    plain = BozolornConfig.from_dict(oracle.make_config(8, 9, [
        oracle.attention_layer(1, 1, 4, 4, 8, 0.5)]))
    assert not is_recurrent(plain)


def test_preset_runs_and_forks_copy_state(tmp_path):
    eng = LLMEngine(EngineConfig.tiny_bozolorn(), device="cpu")
    rid = eng.add_request(list(range(1, 20)),
                          SamplingParams(max_new_tokens=4, temperature=0.0))
    while not eng.is_finished():
        eng.step()
    assert len(eng.get_output(rid).token_ids) == 4
    # every slot buffer of every parallel layer follows a fork
    caches = eng.kv_caches
    leaves = [t for t, kind in caches._all() if kind == "state"]
    assert len(leaves) == 2 * sum(
        l.type == "parallel" for l in eng.cfg.model.layers)
    for t in leaves:
        t[1] = 3
    caches.copy_slot(1, 2)
    assert all(bool((t[2] == 3).all()) for t in leaves)
    # a borrowing layer owns no buffers
    assert caches[3] == ()


def test_local_provider_serves_a_checkpoint_directory(tmp_path):
    """The gateway's local provider with LOCAL_MODEL=hf picks the
    architecture from the directory's config.json and generates through
    the async engine with sampling."""
    import asyncio

    from inference_gateway_amd.config import LocalConfig
    from inference_gateway_amd.providers.local import LocalProvider

    cfg = oracle.make_config(48, 300, [
        oracle.attention_layer(2, 1, 8, 10, 12, 0.35,
                               mlp=oracle.moe_ff(4, 2, 2, 1, 16, 2.0)),
        oracle.parallel_layer(2, 1, 8, 10, 0.35, oracle.rot(4, 100.0),
                              3, 3, 4, 6, 3)], side=4)
    W = oracle.random_weights(cfg, 35)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    lc = LocalConfig(enabled=True, model="hf", max_num_seqs=4,
                     max_model_len=128)
    lc.num_gpu_blocks = 64
    lc.weights_path = path
    provider = LocalProvider(lc, device="cpu")
    try:
        assert isinstance(provider.engine.engine.cfg.model, BozolornConfig)

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


def test_bench_configurations_are_comparable():
    """The speed comparison runs both models at equal width, head sizes
    and active feed-forward size."""
    root = Path(__file__).resolve().parent.parent
    sys.path.insert(0, str(root / "tools"))
    try:
        import bench_bozolorn as bb
    finally:
        sys.path.pop(0)
    for sz in bb.SIZES.values():
        boz, fdi = bb._configs(sz)
        assert boz.hidden_size == fdi.hidden_size == sz["width"]
        assert boz.num_layers == fdi.num_layers
        moe = boz.layers[0].mlp
        assert moe.expert_ff * moe.top == fdi.layers[0].mlp.ff
        a, f = boz.layers[0].mixer.left, fdi.layers[0].mixer.left
        assert (a.heads, a.kv_heads, a.dim, a.vdim) == (
            f.heads, f.kv_heads, f.dim, f.vdim)
        assert boz.layers[3].mixer.kv_from == 1
