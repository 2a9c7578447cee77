#!/usr/bin/env python3
"""Feditar beside Fedatar at equal layer sizes: engine prefill / decode
throughput and per-kernel roofline fractions (random weights).

Run through `python bench.py --arch-compare --arch feditar [--arch-size
NAME]`; prints one JSON object.  Fedatar is the closest model the engine
serves: per-layer mixers (a recurrence or attention over a paged cache)
around an fp32 residual stream, dense feed-forwards, eager decode.  Same
two measurements as tools/bench_hybrid.py: the LLMEngine loop for both
models, and each kernel of the recurrent extension next to the like
kernel of the Fedatar / Llama path, priced against the MI355X roofline
(2.5 PFLOP/s dense bf16, 8 TB/s HBM).  The memory scan runs on the vector
ALU in fp32; its entry also carries the fraction of that unit's peak
(`valu_frac`, 157 TFLOP/s).
"""
from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
sys.path.insert(0, str(Path(__file__).resolve().parent))

from bench_hybrid import _engine_run, _entry, _time  # noqa: E402

PEAK_VALU = 157e12

# Llama-3-8B's layer shape, and a half-width one.  Both models: 4 layers,
# each with a dense feed-forward.
SIZES = {
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128,
               state=128, groups=8, norm_groups=8, ff=14336, vocab=32000,
               layers=4, rdim=64, decay_rank=64,
               kv_rank=512, q_rank=1536, rot_dim=64),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128,
               state=128, groups=4, norm_groups=4, ff=8192, vocab=32000,
               layers=4, rdim=64, decay_rank=32,
               kv_rank=256, q_rank=768, rot_dim=64),
}


def _configs(sz):
    from inference_gateway_amd.engine.config import (
        DecayMemorySpec, LayerSpec, ParallelMixerSpec, fedatar_preset,
        feditar_preset)

    fdi = feditar_preset(
        "feditar-bench", width=sz["width"], vocab=sz["vocab"],
        pattern="xd sd pd pd", heads=sz["heads"], kv_heads=sz["kv_heads"],
        dim=sz["dim"], vdim=sz["vdim"], state=sz["state"],
        groups=sz["groups"], ff=sz["ff"], norm_groups=sz["norm_groups"],
        decay_rank=sz["decay_rank"], max_position=2048)
    # the decayed memory keeps its usual 64 entries per head
    for l in fdi.layers:
        if isinstance(l.mixer, ParallelMixerSpec):
            l.mixer.right = DecayMemorySpec(
                heads=sz["width"] // sz["rdim"], dim=sz["rdim"],
                decay_rank=sz["decay_rank"])
    del LayerSpec
    fda = fedatar_preset(
        "fedatar-bench", width=sz["width"], vocab=sz["vocab"],
        pattern="gd gd ad ad", heads=sz["heads"], dim=sz["dim"],
        rot_dim=sz["rot_dim"], vdim=sz["vdim"], kv_rank=sz["kv_rank"],
        q_rank=sz["q_rank"], window=0, ff=sz["ff"], experts=1, top=1,
        expert_ff=sz["ff"], shared_ff=0)
    return fdi, fda


def _scan_entry(t, T, H, N, P, in_bytes):
    """4 useful FLOP per (row, head, key entry, column): update and
    read-out; the kernel spends 6 (k v as its own product)."""
    e = _entry(t, flops=4.0 * T * H * N * P, bytes_=in_bytes)
    e["valu_frac"] = round(6.0 * T * H * N * P / t / PEAK_VALU, 4)
    return e


def _kernels(sz):
    from inference_gateway_amd import ops

    dev, bf = "cuda", torch.bfloat16
    D, H, G = sz["width"], sz["heads"], sz["kv_heads"]
    N, P = sz["dim"], sz["vdim"]
    out = {}
    bs = 16

    def seqs(nseq, L, start):
        T = nseq * L
        cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
        st = torch.full((nseq,), start, dtype=torch.int32, device=dev)
        sl = torch.arange(nseq, dtype=torch.int32, device=dev)
        rs = sl.repeat_interleave(L)
        return T, cu, st, sl, rs

    # ---- attention: 4 x 2048 prompt rows; 256 decoded rows at 2048 ----
    def paged(nseq, ctx):
        nb = nseq * (ctx // bs) + 1
        kc = torch.randn(nb, G, bs, N, device=dev, dtype=bf)
        vc = torch.randn(nb, G, bs, P, device=dev, dtype=bf)
        bt = (torch.arange(nseq * (ctx // bs), dtype=torch.int32,
                           device=dev) + 1).view(nseq, ctx // bs)
        return kc, vc, bt

    nseq, L = 4, 2048
    T, cu, st, sl, row_seq = seqs(nseq, L, 0)
    kc, vc, bt = paged(nseq, L)
    q = torch.randn(T, H * N, device=dev, dtype=bf)
    pos = torch.arange(L, dtype=torch.int32, device=dev).repeat(nseq)
    keys = nseq * L * (L + 1) / 2
    t = _time(lambda: ops.softcap_attention(
        q, kc, vc, bt, row_seq, pos, 0.09, 50.0, 0.1, 128, 0, T, [L] * nseq,
        cu, st), 3)
    out["softcap_attention_prompt"] = _entry(t, flops=2.0 * keys * H
                                             * (N + P))
    hd = 128
    q3 = torch.randn(T, H, hd, device=dev, dtype=bf)
    k3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    v3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    t = _time(lambda: ops.flash_prefill(q3, k3, v3, cu, [L] * nseq, 0.09), 5)
    out["flash_prefill"] = _entry(t, flops=4.0 * keys * H * hd)
    B, ctx = 256, 2048
    kc, vc, bt = paged(B, ctx)
    q = torch.randn(B, H * N, device=dev, dtype=bf)
    rs1 = torch.arange(B, dtype=torch.int32, device=dev)
    pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)
    cu1 = torch.arange(B + 1, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.softcap_attention(
        q, kc, vc, bt, rs1, pos, 0.09, 50.0, 0.1, 128, 0, 0, None, cu1,
        pos), 5)
    out["softcap_attention_decode"] = _entry(
        t, flops=2.0 * B * ctx * H * (N + P),
        bytes_=2.0 * B * ctx * G * (N + P))
    kc2 = torch.randn(B * (ctx // bs) + 1, G, bs, hd, device=dev, dtype=bf)
    vc2 = torch.randn_like(kc2)
    ctx_lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q3 = torch.randn(B, H, hd, device=dev, dtype=bf)
    t = _time(lambda: ops.paged_attn_decode(q3, kc2, vc2, bt, ctx_lens, 0.09))
    out["paged_attn_decode"] = _entry(
        t, flops=4.0 * B * ctx * H * hd, bytes_=4.0 * B * ctx * G * hd)
    del kc, vc, kc2, vc2

    # ---- memory scans: 64 x 1024 prompt rows; 256 decoded rows ----
    RH, RN = D // sz["rdim"], sz["rdim"]
    for tag, nseq, L, start in (("prompt", 64, 1024, 0),
                                ("decode", 256, 1, 5)):
        T, cu, st, sl, row_seq = seqs(nseq, L, start)
        it = 3 if L > 1 else 20
        # matrix memory: scalar decay, normaliser column
        qk = torch.randn(T, 2, H, N, device=dev, dtype=bf)
        v = torch.randn(T, H, P, device=dev, dtype=bf)
        a = torch.rand(T, H, 1, device=dev)
        c = torch.rand(T, H, device=dev)
        mem = torch.zeros(nseq, H * N * (P + 1), device=dev)
        t = _time(lambda: ops.outer_scan(
            qk[:, 0], qk[:, 1], v, a, c, None, None, mem, cu, st, sl,
            [L] * nseq, ops.DECAY_LINEAR, True, 0.1), it)
        io = T * H * (2 * N + P) * 2.0 + T * H * (P + 1) * 4.0 \
            + 2.0 * mem.numel() * 4
        out[f"outer_scan_mlstm_{tag}"] = _scan_entry(t, T, H, N, P, io)
        # state space: grouped B / C, skip
        Ns = sz["state"]
        bc = torch.randn(T, 2, sz["groups"], Ns, device=dev, dtype=bf)
        mem = torch.zeros(nseq, H * Ns * P, device=dev)
        skip = torch.ones(H, device=dev)
        t = _time(lambda: ops.outer_scan(
            bc[:, 1], bc[:, 0], v, a, c, None, skip, mem, cu, st, sl,
            [L] * nseq, ops.DECAY_LINEAR, False, 1.0), it)
        io = T * (2 * sz["groups"] * Ns + H * P) * 2.0 + T * H * P * 4.0 \
            + 2.0 * mem.numel() * 4
        out[f"outer_scan_ssm_{tag}"] = _scan_entry(t, T, H, Ns, P, io)
        # decayed memory: per-entry decay, bonus
        rkv = torch.randn(3, T, RH, RN, device=dev, dtype=bf)
        lw = torch.randn(T, RH, RN, device=dev) - 1.0
        u = torch.randn(RH, RN, device=dev)
        mem = torch.zeros(nseq, RH * RN * RN, device=dev)
        t = _time(lambda: ops.outer_scan(
            rkv[0], rkv[1], rkv[2], lw, None, u, None, mem, cu, st, sl,
            [L] * nseq, ops.DECAY_EXP_NEG_EXP, False, 1.0), it)
        io = T * RH * RN * (3 * 2.0 + 4 + 4) + 2.0 * mem.numel() * 4
        out[f"outer_scan_decay_{tag}"] = _scan_entry(t, T, RH, RN, RN, io)
        # the like kernel: Fedatar's gated recurrence over the width
        zug = torch.randn(T, 3 * D, device=dev, dtype=bf)
        state = torch.zeros(nseq, D, device=dev)
        t = _time(lambda: ops.mingru_scan(zug, state, cu, st, sl,
                                          [L] * nseq), it)
        out[f"mingru_scan_{tag}"] = _entry(
            t, bytes_=T * D * ((2 * 6 + 2.0) if L > 1 else 8.0)
            + 2.0 * state.numel() * 4)
        # gates and the read-out epilogue
        pre = torch.randn(T, 2 * H, device=dev)
        ms = torch.zeros(nseq, H, device=dev)
        t = _time(lambda: ops.mlstm_gates(pre, 15.0, ms, cu, st, sl), it)
        out[f"mlstm_gates_{tag}"] = _entry(t, bytes_=T * H * 20.0)
        o = torch.randn(T, H, P, device=dev)
        dn = torch.randn(T, H, device=dev)
        gate = torch.randn(T, H * P, device=dev, dtype=bf)
        w = torch.ones(H * P, device=dev)
        fl = torch.rand(T, H, device=dev)
        t = _time(lambda: ops.head_norm_gate(o, gate, w, 1e-6, P,
                                             ops.GATE_SIGMOID, False, dn,
                                             fl, bf), it)
        out[f"head_norm_gate_{tag}"] = _entry(
            t, bytes_=T * H * (P * 4.0 + 8 + P * 4.0))

    # ---- row kernels on 8192 rows (8 sequences of 1024) ----
    T, cu, st, sl, row_seq = seqs(8, 1024, 0)
    res = torch.randn(T, D, device=dev)
    dl = torch.randn(T, D, device=dev, dtype=bf)
    w = torch.ones(D, device=dev)
    t = _time(lambda: ops.add_rmsnorm_pair(res, dl, None, w, None, 1e-6, bf))
    out["add_rmsnorm"] = _entry(t, bytes_=T * D * (4 + 4 + 2 + 2.0))
    t = _time(lambda: ops.add_layernorm(res, dl, w, w, 1e-5, bf))
    out["add_layernorm"] = _entry(t, bytes_=T * D * (4 + 4 + 2 + 2.0))
    x = torch.randn(T, D, device=dev, dtype=bf)
    rsd = torch.randn(T, D, device=dev, dtype=bf)
    wb = torch.ones(D, device=dev, dtype=bf)
    t = _time(lambda: ops.fused_add_rmsnorm(x, rsd, wb, 1e-5))
    out["fused_add_rmsnorm"] = _entry(t, bytes_=T * D * 8.0)
    t = _time(lambda: ops.rmsnorm_pair_mean(x, rsd, w, w, 1e-6))
    out["rmsnorm_pair_mean"] = _entry(t, bytes_=T * D * 6.0)
    tok = torch.randint(0, sz["vocab"], (T,), device=dev)
    pos = torch.arange(1024, dtype=torch.int32, device=dev).repeat(8)
    emb = torch.randn(sz["vocab"], D, device=dev, dtype=bf)
    pair = torch.randn(4094, D, device=dev, dtype=bf)
    ptab = torch.randn(1024, D, device=dev, dtype=bf)
    prev = torch.zeros(8, 1, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.embed_pair_norm(
        tok, pos, prev, cu, st, sl, row_seq, emb, pair, ptab, w, 64.0, 4093,
        8191, 131, 1e-6))
    out["embed_pair_norm"] = _entry(t, bytes_=T * D * (6 + 4.0))
    mu = torch.rand(5, D, device=dev)
    hs = torch.zeros(8, D, device=dev)
    t = _time(lambda: ops.token_shift_mix(x, mu, hs, cu, st, sl, row_seq))
    out["token_shift_mix"] = _entry(t, bytes_=T * D * (2 + 10.0))
    C = H * N + G * N + G * P
    proj = torch.randn(T, C, device=dev, dtype=bf)
    cw = torch.randn(C, 4, device=dev)
    cs = torch.zeros(8, 3 * C, device=dev)
    t = _time(lambda: ops.causal_conv(proj, cw, None, cs, cu, st, sl,
                                      row_seq, False))
    out["causal_conv"] = _entry(t, bytes_=T * C * 4.0)
    kcs = torch.zeros(T // bs + 1, G, bs, N, device=dev, dtype=bf)
    vcs = torch.zeros(T // bs + 1, G, bs, P, device=dev, dtype=bf)
    slots = torch.arange(bs, T + bs, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.append_paged_kv(
        proj[:, H * N:H * N + G * N], proj[:, H * N + G * N:], kcs, vcs,
        slots))
    out["append_paged_kv"] = _entry(t, bytes_=T * G * (N + P) * 4.0)
    k3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    v3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    kc2 = torch.zeros(T // bs + 1, G, bs, hd, device=dev, dtype=bf)
    vc2 = torch.zeros_like(kc2)
    t = _time(lambda: ops.append_kv_cache(k3, v3, kc2, vc2, slots))
    out["append_kv_cache"] = _entry(t, bytes_=T * G * hd * 8.0)

    # ---- activations on [8192, ff] ----
    F_ = sz["ff"]
    z = torch.randn(T, F_, device=dev, dtype=bf)
    t = _time(lambda: ops.relu2(z))
    out["relu2"] = _entry(t, bytes_=T * F_ * 4.0)
    gu = torch.randn(T, 2 * F_, device=dev, dtype=bf)
    t = _time(lambda: ops.silu_mul(gu))
    out["silu_mul"] = _entry(t, bytes_=T * F_ * 6.0)
    return out


def run(size: str = "2k", batch: int = 64, prompt_len: int = 1024,
        steps: int = 32, warmup: int = 4) -> dict:
    sz = SIZES[size]
    fdi, fda = _configs(sz)
    res = {"size": size, "shape": sz, "batch": batch,
           "prompt_len": prompt_len, "steps": steps, "dtype": "bf16",
           "data": "synthetic (random weights and tokens)"}
    res["kernels"] = _kernels(sz)
    res["feditar"] = _engine_run(fdi, batch, prompt_len, steps, warmup)
    res["fedatar"] = _engine_run(fda, batch, prompt_len, steps, warmup)
    return res


if __name__ == "__main__":
    print(json.dumps(run(*(sys.argv[1:2] or ["2k"]))))
