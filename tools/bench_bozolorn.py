#!/usr/bin/env python3
"""Bozolorn beside Feditar at equal layer sizes: engine prefill / decode
throughput and per-kernel roofline fractions (random weights).

Run through `python bench.py --arch-compare --arch bozolorn [--arch-size
NAME]`; prints one JSON object.  Feditar is the closest model the engine
serves: a parallel mixer of paged softmax attention beside an
outer-product memory, an fp32 residual stream, eager decode, the same
kernel extension.  Both models get 4 layers of the same width, head
counts and head sizes; Bozolorn's experts are sized so that the `top`
chosen ones together equal Feditar's dense feed-forward.  Same two
measurements as tools/bench_recurrent.py: the LLMEngine loop for both
models, and each new kernel next to the like kernel of the Feditar /
Mekevik path, priced against the MI355X roofline (2.5 PFLOP/s dense bf16,
8 TB/s HBM).  The memory scans run on the vector ALU in fp32; their
entries also carry the fraction of that unit's peak (`valu_frac`, 157
TFLOP/s).
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

# Llama-3-8B's layer shape, and a half-width one
SIZES = {
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128,
               ff=14336, vocab=32000, experts=8, top=2, groups=4, keep=2,
               chunk=1024, rot_dims=64, side=64, decay_rank=64, state=128),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128,
               ff=8192, vocab=32000, experts=8, top=2, groups=4, keep=2,
               chunk=1024, rot_dims=64, side=64, decay_rank=32, state=128),
}


def _configs(sz):
    from inference_gateway_amd.engine.config import (bozolorn_preset,
                                                     feditar_preset)

    boz = bozolorn_preset(
        "bozolorn-bench", width=sz["width"], vocab=sz["vocab"],
        pattern="pm am pm a1m", heads=sz["heads"], kv_heads=sz["kv_heads"],
        dim=sz["dim"], vdim=sz["vdim"], chunk=sz["chunk"],
        rot_dims=sz["rot_dims"], d_heads=sz["heads"],
        d_kv_heads=sz["kv_heads"], d_dim=sz["dim"], d_vdim=sz["vdim"],
        experts=sz["experts"], top=sz["top"], groups=sz["groups"],
        keep=sz["keep"], expert_ff=sz["ff"] // sz["top"],
        side_dim=sz["side"], yarn_factor=4.0, yarn_original=4096.0)
    fdi = feditar_preset(
        "feditar-bench", width=sz["width"], vocab=sz["vocab"],
        pattern="pd pd pd pd", heads=sz["heads"], kv_heads=sz["kv_heads"],
        dim=sz["dim"], vdim=sz["vdim"], state=sz["state"], groups=1,
        ff=sz["ff"], decay_rank=sz["decay_rank"], max_position=2048)
    return boz, fdi


def _scan_entry(t, T, H, N, P, in_bytes, issued):
    """4 useful FLOP per (row, head, key entry, column): update and
    read-out; `issued` = what the kernel spends."""
    e = _entry(t, flops=4.0 * T * H * N * P, bytes_=in_bytes)
    e["valu_frac"] = round(issued * T * H * N * P / t / PEAK_VALU, 4)
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

    def paged(nseq, ctx):
        nb = nseq * (ctx // bs) + 1
        kc = torch.randn(nb, G, bs, N, device=dev, dtype=bf)
        vc = torch.randn(nb, G, bs, P, device=dev, dtype=bf)
        bt = (torch.arange(nseq * (ctx // bs), dtype=torch.int32,
                           device=dev) + 1).view(nseq, ctx // bs)
        return kc, vc, bt

    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
                          device=dev)
    sinks = torch.zeros(H, device=dev)
    chunk = sz["chunk"]

    # ---- attention: 4 x 2048 prompt rows; 256 decoded rows at 2048 ----
    nseq, L = 4, 2048
    T, cu, st, sl, row_seq = seqs(nseq, L, 0)
    kc, vc, bt = paged(nseq, L)
    q = torch.randn(T, H * N, device=dev, dtype=bf)
    gate = torch.randn(T, H * P, device=dev, dtype=bf)
    pos = torch.arange(L, dtype=torch.int32, device=dev).repeat(nseq)
    keys = nseq * L * (L + 1) / 2
    ckeys = nseq * sum(p % chunk + 1 for p in range(L))
    base = (q, kc, vc, bt, row_seq, pos, 0.09)
    tail = (0, T, [L] * nseq, cu, st)
    t = _time(lambda: ops.softcap_attention(*base, 0.0, 0.0, 1, *tail,
                                            sinks=sinks), 3)
    out["sink_attention_prompt"] = _entry(t, flops=2.0 * keys * H * (N + P))
    t = _time(lambda: ops.softcap_attention(
        *base, 0.0, 0.0, 1, *tail, slopes=slopes, chunk=chunk, gate=gate), 3)
    out["chunk_bias_attention_prompt"] = _entry(
        t, flops=2.0 * ckeys * H * (N + P))
    t = _time(lambda: ops.softcap_attention(*base, 50.0, 0.1, 128, *tail), 3)
    out["softcap_attention_prompt"] = _entry(t, flops=2.0 * keys * H
                                             * (N + P))
    B, ctx = 256, 2048
    kc, vc, bt = paged(B, ctx)
    q = torch.randn(B, H * N, device=dev, dtype=bf)
    gate = torch.randn(B, H * P, device=dev, dtype=bf)
    rs1 = torch.arange(B, dtype=torch.int32, device=dev)
    pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)
    cu1 = torch.arange(B + 1, dtype=torch.int32, device=dev)
    base = (q, kc, vc, bt, rs1, pos, 0.09)
    tail = (0, 0, None, cu1, pos)
    dkeys = (ctx - 1) % chunk + 1
    t = _time(lambda: ops.softcap_attention(*base, 0.0, 0.0, 1, *tail,
                                            sinks=sinks), 5)
    out["sink_attention_decode"] = _entry(
        t, flops=2.0 * B * ctx * H * (N + P),
        bytes_=2.0 * B * ctx * G * (N + P))
    t = _time(lambda: ops.softcap_attention(
        *base, 0.0, 0.0, 1, *tail, slopes=slopes, chunk=chunk, gate=gate), 5)
    out["chunk_bias_attention_decode"] = _entry(
        t, flops=2.0 * B * dkeys * H * (N + P),
        bytes_=2.0 * B * dkeys * G * (N + P))
    t = _time(lambda: ops.softcap_attention(*base, 50.0, 0.1, 128, *tail), 5)
    out["softcap_attention_decode"] = _entry(
        t, flops=2.0 * B * ctx * H * (N + P),
        bytes_=2.0 * B * ctx * G * (N + P))
    del kc, vc

    # ---- memory scans: 64 x 1024 prompt rows; 256 decoded rows ----
    for tag, nseq, L, start in (("prompt", 64, 1024, 0),
                                ("decode", 256, 1, 5)):
        T, cu, st, sl, row_seq = seqs(nseq, L, start)
        it = 3 if L > 1 else 20
        qk = torch.randn(T, 2, G, N, device=dev, dtype=bf)
        v = torch.randn(T, H, P, device=dev, dtype=bf)
        a = torch.rand(T, H, device=dev) * 0.5 + 0.5
        b = torch.rand(T, H, device=dev)
        mem = torch.zeros(nseq, H * N * P, device=dev)
        t = _time(lambda: ops.delta_scan(
            qk[:, 0], qk[:, 1], v, a, b, mem, cu, st, sl, [L] * nseq, 1e-6,
            N ** -0.5), it)
        io = T * (2 * G * N + H * P) * 2.0 + T * H * (P * 4.0 + 8) \
            + 2.0 * mem.numel() * 4
        out[f"delta_scan_{tag}"] = _scan_entry(t, T, H, N, P, io, 8.0)
        # the like kernel: Feditar's scalar-decay outer-product memory at
        # the same head sizes
        a3 = a.unsqueeze(-1).contiguous()
        mem2 = torch.zeros(nseq, H * N * P, device=dev)
        t = _time(lambda: ops.outer_scan(
            qk[:, 0], qk[:, 1], v, a3, b, None, None, mem2, cu, st, sl,
            [L] * nseq, ops.DECAY_LINEAR, False, 1.0), it)
        out[f"outer_scan_{tag}"] = _scan_entry(t, T, H, N, P, io, 6.0)
        pre = torch.randn(T, 2 * H, device=dev)
        al = torch.zeros(H, device=dev)
        t = _time(lambda: ops.decay_beta_gates(pre, al, al), it)
        out[f"decay_beta_gates_{tag}"] = _entry(t, bytes_=T * H * 16.0)
        t = _time(lambda: ops.ssm_gates(pre[:, :H].contiguous(), al), it)
        out[f"ssm_gates_{tag}"] = _entry(t, bytes_=T * H * 12.0)
        o = torch.randn(T, H, P, device=dev)
        g2 = torch.randn(T, H * P, device=dev, dtype=bf)
        w = torch.ones(H * P, device=dev)
        t = _time(lambda: ops.head_norm_gate(o, g2, w, 1e-6, P,
                                             ops.GATE_SILU, False, None,
                                             None, bf), it)
        out[f"head_norm_gate_{tag}"] = _entry(
            t, bytes_=T * H * P * (4.0 + 2 + 2))

    # ---- row kernels on 8192 rows (8 sequences of 1024) ----
    T, cu, st, sl, row_seq = seqs(8, 1024, 0)
    res = torch.randn(T, D, device=dev)
    dl = torch.randn(T, D, device=dev, dtype=bf)
    w = torch.ones(D, device=dev)
    t = _time(lambda: ops.add_normed_rmsnorm(res, dl, w, w, 1e-6, bf))
    out["add_normed_rmsnorm"] = _entry(t, bytes_=T * D * (4 + 4 + 2 + 2.0))
    t = _time(lambda: ops.add_rmsnorm_pair(res, dl, None, w, None, 1e-6, bf))
    out["add_rmsnorm"] = _entry(t, bytes_=T * D * (4 + 4 + 2 + 2.0))
    C = H * N + G * N + G * P
    proj = torch.randn(T, C, device=dev, dtype=bf)
    pos = torch.arange(1024, dtype=torch.int32, device=dev).repeat(8)
    kcs = torch.zeros(T // bs + 1, G, bs, N, device=dev, dtype=bf)
    vcs = torch.zeros(T // bs + 1, G, bs, P, device=dev, dtype=bf)
    slots = torch.arange(bs, T + bs, dtype=torch.int32, device=dev)
    wn = torch.ones(N, device=dev)
    inv = torch.rand(sz["rot_dims"] // 2, device=dev)
    t = _time(lambda: ops.qk_norm_rope_append(
        proj, pos, slots, kcs, vcs, wn, wn, inv, 1.1, 1e-6, H, G, N, P))
    out["qk_norm_rope_append"] = _entry(t, bytes_=T * C * 4.0)
    t = _time(lambda: ops.append_paged_kv(
        proj[:, H * N:H * N + G * N], proj[:, H * N + G * N:], kcs, vcs,
        slots))
    out["append_paged_kv"] = _entry(t, bytes_=T * G * (N + P) * 4.0)
    if ops.HAS_HYBRID:
        # the like kernel: Mekevik's norm over the whole q and k blocks +
        # append (page-transposed values)
        vct = torch.zeros(T // bs + 1, G, P, bs, device=dev, dtype=bf)
        wq, wk = torch.ones(H * N, device=dev), torch.ones(G * N, device=dev)
        t = _time(lambda: ops.qk_norm_append(proj, slots, kcs, vct, wq, wk,
                                             None, 0.0, 1e-6, H, G, N, P))
        out["qk_norm_append"] = _entry(t, bytes_=T * C * 4.0)
    CC = 2 * G * N + H * P
    pj = torch.randn(T, CC + H * P, device=dev, dtype=bf)
    cw = torch.randn(CC, 4, device=dev)
    cs = torch.zeros(8, 3 * CC, device=dev)
    t = _time(lambda: ops.causal_conv(pj[:, :CC], cw, None, cs, cu, st, sl,
                                      row_seq, True))
    out["causal_conv_silu"] = _entry(t, bytes_=T * CC * 4.0)
    sd = sz["side"]
    z = torch.randn(T, sd, device=dev, dtype=bf)
    table = torch.randn(sz["vocab"], 4 * sd, device=dev, dtype=bf)
    tok = torch.randint(0, sz["vocab"], (T,), device=dev)
    t = _time(lambda: ops.gelu_mul_rows(z, table, tok, sd))
    out["gelu_mul_rows"] = _entry(t, bytes_=T * sd * 6.0)

    # ---- expert activation on [8192 * top, expert ff] and routing ----
    F_ = sz["ff"] // sz["top"]
    gu = torch.randn(T * sz["top"], 2 * F_, device=dev, dtype=bf)
    t = _time(lambda: ops.gated_act(gu, ops.GATED_ACT_CLAMPED, 7.0, 1.702))
    out["gated_act_clamped"] = _entry(t, bytes_=T * sz["top"] * F_ * 6.0)
    z2 = torch.randn(T, sz["ff"], device=dev, dtype=bf)
    t = _time(lambda: ops.relu2(z2))
    out["relu2"] = _entry(t, bytes_=T * sz["ff"] * 4.0)
    for rows in (256, 8192):
        lg = torch.randn(rows, sz["experts"], device=dev)
        corr = torch.zeros(sz["experts"], device=dev)
        t = _time(lambda: ops.moe_group_route(
            lg, corr, sz["top"], sz["groups"], sz["keep"],
            rows if rows <= 256 else 0))
        out[f"moe_group_route_{rows}"] = _entry(
            t, bytes_=rows * (sz["experts"] * 4.0 + sz["top"] * 16.0))
        if ops.HAS_HYBRID:
            t = _time(lambda: ops.moe_topk_route(
                lg, sz["top"], rows if rows <= 256 else 0))
            out[f"moe_topk_route_{rows}"] = _entry(
                t, bytes_=rows * (sz["experts"] * 4.0 + sz["top"] * 16.0))
    return out


def run(size: str = "2k", batch: int = 64, prompt_len: int = 1024,
        steps: int = 32, warmup: int = 4) -> dict:
    sz = SIZES[size]
    boz, fdi = _configs(sz)
    res = {"size": size, "shape": sz, "batch": batch,
           "prompt_len": prompt_len, "steps": steps, "dtype": "bf16",
           "data": "synthetic (random weights and tokens)"}
    res["kernels"] = _kernels(sz)
    res["bozolorn"] = _engine_run(boz, batch, prompt_len, steps, warmup)
    res["feditar"] = _engine_run(fdi, batch, prompt_len, steps, warmup)
    return res


if __name__ == "__main__":
    print(json.dumps(run(*(sys.argv[1:2] or ["2k"]))))
