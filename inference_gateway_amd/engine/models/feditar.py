"""Feditar: a per-layer decoder of recurrent mixers for the MI355X engine.

The fp32 residual stream starts as the normed sum of a scaled token row,
a hashed (previous, current) token-pair row and a learned position row.
Every layer is pre-norm (RMS, weight stored around zero) around one MIXER
and, optionally, a relu^2 feed-forward, chosen per layer:

  MLSTMMixer        matrix memory with stabilised exponential gates
  Mamba2Mixer       state-space layer: short convolution, scalar decay
                    per head, gated grouped norm
  ParallelMixer     SoftcapAttention (short convolutions on q/k/v,
                    position-dependent query stretch, tanh score cap,
                    grouped heads; pages K and V) beside DecayMemory
                    (token-shift mixes, low-rank per-channel decays,
                    look-before-write outer-product memory); the two
                    outputs are normed over the width and averaged

All three memories are ONE recurrence, S' = diag(a) S + (c k) v^T read
with a query, and run on one kernel (ops.outer_scan); what differs is how
a, c, k, q are made and the read-out's epilogue (ops.head_norm_gate).
Everything a layer keeps between steps is a slot buffer or paged K/V
handed in by the engine (cache_specs), so portions of prompts, decoded
tokens and mixed batches are the same code path.  GEMMs go through
F.linear/bmm; the small projections that feed gates, step sizes and
decays run in fp32.
"""
from __future__ import annotations

from typing import List

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import ops
from ...parallel.comm import tp_world_size
from ..config import (DecayMemorySpec, FeditarConfig, Mamba2Spec, MLSTMSpec,
                      ParallelMixerSpec, SoftcapAttentionSpec)
from .batch import ForwardBatch
from .fedatar import _param, _rand


def _w(shape, device, dtype, name, fan_in):
    return _param(_rand(shape, device, dtype, name, fan_in ** -0.5 / 0.02))


def _one_plus(n, device, name):
    """A norm weight stored around zero, held as 1 + w in fp32."""
    return _param(1.0 + _rand((n,), device, torch.float32, name, 5.0))


class MLSTMMixer(nn.Module):
    """q = W_q h N^-1/2, k = W_k h, v = W_v h; per head log gates i =
    cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)); running maximum
    m (0 at the start); S <- e^(f + m_prev - m) S + e^(i - m) k v^T with a
    normaliser column n; o = S^T q / (max(|n . q|, e^-m) + 1e-6); per-head
    RMS norm, weight, sigmoid(W_g h) gate, W_o."""

    def __init__(self, hidden: int, spec: MLSTMSpec, eps: float, name: str,
                 device, dtype):
        super().__init__()
        self.spec, self.eps, self.dtype = spec, eps, dtype
        H, N, P = spec.heads, spec.dim, spec.vdim
        # fused input projection: q | k | v | output-gate logits
        self.qkvg = _w((2 * H * N + 2 * H * P, hidden), device, dtype,
                       name + ".qkvg", hidden)
        # input | forget gate logits, fp32
        self.gates_w = _w((2 * H, hidden), device, torch.float32,
                          name + ".if", hidden)
        self.gates_b = _param(_rand((2 * H,), device, torch.float32,
                                    name + ".if_b", 50.0))
        self.norm_w = _param(1.0 + _rand((H * P,), device, torch.float32,
                                         name + ".norm", 5.0))
        self.o = _w((hidden, H * P), device, dtype, name + ".o", H * P)

    def cache_spec(self):
        s = self.spec
        return ("group", [("state", s.heads * s.dim * (s.vdim + 1)),
                          ("state", s.heads)])

    def forward(self, h, fb: ForwardBatch, cache):
        mem, m_state = cache
        s = self.spec
        H, N, P = s.heads, s.dim, s.vdim
        T = h.shape[0]
        proj = F.linear(h, self.qkvg)
        pre = F.linear(h.float(), self.gates_w, self.gates_b)
        decay, kscale, floor = ops.mlstm_gates(
            pre, s.gate_cap, m_state, fb.seq_cu, fb.seq_start, fb.seq_slots)
        o, den = ops.outer_scan(
            proj[:, :H * N].view(T, H, N),
            proj[:, H * N:2 * H * N].view(T, H, N),
            proj[:, 2 * H * N:2 * H * N + H * P].view(T, H, P),
            decay.unsqueeze(-1), kscale, None, None, mem, fb.seq_cu,
            fb.seq_start, fb.seq_slots, fb.seq_rows, ops.DECAY_LINEAR,
            True, float(N) ** -0.5)
        y = ops.head_norm_gate(o, proj[:, 2 * H * N + H * P:], self.norm_w,
                               self.eps, P, ops.GATE_SIGMOID, False, den,
                               floor, self.dtype)
        return F.linear(y, self.o)


class Mamba2Mixer(nn.Module):
    """W_in h = [z | x | B | C | dt]; x, B, C through a short causal
    convolution (bias) and silu; dt = softplus(dt + bias); per head S <-
    e^(-e^A dt) S + dt B x^T, y = S^T C + D x; y silu(z), RMS norm in
    equal parts, weight, W_o."""

    def __init__(self, hidden: int, spec: Mamba2Spec, eps: float, name: str,
                 device, dtype):
        super().__init__()
        self.spec, self.eps, self.dtype = spec, eps, dtype
        H, inner, CC = spec.heads, spec.inner, spec.conv_channels
        # z | x | B | C rows of the input projection; the dt rows run
        # apart in fp32
        self.in_main = _w((inner + CC, hidden), device, dtype,
                          name + ".in", hidden)
        self.dt_w = _w((H, hidden), device, torch.float32, name + ".dt",
                       hidden)
        self.dt_b = _param(_rand((H,), device, torch.float32,
                                 name + ".dt_b", 50.0))
        self.conv_w = _param(_rand((CC, spec.conv), device, torch.float32,
                                   name + ".conv", 25.0))
        self.conv_b = _param(_rand((CC,), device, torch.float32,
                                   name + ".conv_b", 5.0))
        self.a_log = _param(_rand((H,), device, torch.float32,
                                  name + ".a_log", 25.0))
        self.skip = _param(1.0 + _rand((H,), device, torch.float32,
                                       name + ".skip", 5.0))
        self.norm_w = _param(1.0 + _rand((inner,), device, torch.float32,
                                         name + ".norm", 5.0))
        self.o = _w((hidden, inner), device, dtype, name + ".o", inner)

    def cache_spec(self):
        s = self.spec
        return ("group", [("state", (s.conv - 1) * s.conv_channels),
                          ("state", s.heads * s.state * s.vdim)])

    def forward(self, h, fb: ForwardBatch, cache):
        conv_state, mem = cache
        s = self.spec
        H, P, N, G, inner = s.heads, s.vdim, s.state, s.groups, s.inner
        T = h.shape[0]
        proj = F.linear(h, self.in_main)
        decay, dt = ops.ssm_gates(
            F.linear(h.float(), self.dt_w, self.dt_b), self.a_log)
        xbc = ops.causal_conv(proj[:, inner:], self.conv_w, self.conv_b,
                              conv_state, fb.seq_cu, fb.seq_start,
                              fb.seq_slots, fb.row_seq, True)
        o, _ = ops.outer_scan(
            xbc[:, inner + G * N:].view(T, G, N),
            xbc[:, inner:inner + G * N].view(T, G, N),
            xbc[:, :inner].view(T, H, P), decay.unsqueeze(-1), dt, None,
            self.skip, mem, fb.seq_cu, fb.seq_start, fb.seq_slots,
            fb.seq_rows, ops.DECAY_LINEAR, False, 1.0)
        y = ops.head_norm_gate(o, proj[:, :inner], self.norm_w, self.eps,
                               inner // s.norm_groups, ops.GATE_SILU, True,
                               None, None, self.dtype)
        return F.linear(y, self.o)


class SoftcapAttention(nn.Module):
    """Causal softmax attention without rotation: q, k, v each pass a
    short per-channel causal convolution right after their projection;
    the score is (q . k) scale temp(p) through cap tanh(. / cap), where
    temp(p) = 1 + coef ln(floor((p + 1) / every) + 1) stretches the query
    with its position; grouped heads, own value width."""

    def __init__(self, hidden: int, spec: SoftcapAttentionSpec, name: str,
                 device, dtype):
        super().__init__()
        self.spec = spec
        H, G, N, P = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        self.channels = H * N + G * N + G * P
        self.qkv = _w((self.channels, hidden), device, dtype, name + ".qkv",
                      hidden)
        self.conv_w = _param(_rand((self.channels, spec.conv), device,
                                   torch.float32, name + ".conv", 25.0))
        self.o = _w((hidden, H * P), device, dtype, name + ".o", H * P)

    def cache_spec(self):
        s = self.spec
        return [("paged_k_v", s.kv_heads, s.dim, s.vdim),
                ("state", max(1, (s.conv - 1) * self.channels))]

    def forward(self, h, fb: ForwardBatch, cache):
        (kc, vc), conv_state = cache
        s = self.spec
        HN, GN = s.heads * s.dim, s.kv_heads * s.dim
        c = F.linear(h, self.qkv)
        if s.conv > 1:
            c = ops.causal_conv(c, self.conv_w, None, conv_state, fb.seq_cu,
                                fb.seq_start, fb.seq_slots, fb.row_seq,
                                False)
        ops.append_paged_kv(c[:, HN:HN + GN], c[:, HN + GN:], kc, vc,
                            fb.slot_mapping)
        o = ops.softcap_attention(
            c[:, :HN], kc, vc, fb.seq_block_table, fb.row_seq, fb.positions,
            s.scale, s.softcap, s.temp_coef, s.temp_every, 0,
            fb.num_chunk_rows, fb.seq_lens, fb.seq_cu, fb.seq_start)
        return F.linear(o, self.o)


class DecayMemory(nn.Module):
    """RWKV-style time mixing: r, k, v, g, w each read their own blend
    of h and the previous token's h; per-channel decay a = exp(-exp(W_2
    tanh(W_1 mix_w) + w_0)); o = (S + diag(u) k v^T)^T r, then S <-
    diag(a) S + k v^T; per-head RMS norm, weight, silu gate, W_o."""

    MIXES = "rkvgw"

    def __init__(self, hidden: int, spec: DecayMemorySpec, eps: float,
                 name: str, device, dtype):
        super().__init__()
        self.spec, self.eps, self.dtype = spec, eps, dtype
        H, N, R = spec.heads, spec.dim, spec.decay_rank
        self.hidden = hidden
        self.mu = _param(0.5 + _rand((5, hidden), device, torch.float32,
                                     name + ".mu", 10.0))
        # r | k | v | g projections, K-major for one batched GEMM
        self.rkvg_t = _w((4, hidden, H * N), device, dtype, name + ".rkvg",
                         hidden)
        self.w1 = _w((R, hidden), device, torch.float32, name + ".w1",
                     hidden)
        self.w2 = _w((H * N, R), device, torch.float32, name + ".w2", R)
        self.w0 = _param(-1.0 + _rand((H * N,), device, torch.float32,
                                      name + ".w0", 25.0))
        self.bonus = _param(_rand((H, N), device, torch.float32,
                                  name + ".u", 25.0))
        self.norm_w = _param(1.0 + _rand((H * N,), device, torch.float32,
                                         name + ".norm", 5.0))
        self.o = _w((hidden, H * N), device, dtype, name + ".o", H * N)

    def cache_spec(self):
        s = self.spec
        return [("state", self.hidden),
                ("state", s.heads * s.dim * s.dim)]

    def forward(self, h, fb: ForwardBatch, cache):
        prev_h, mem = cache
        s = self.spec
        H, N = s.heads, s.dim
        T = h.shape[0]
        mixes = ops.token_shift_mix(h, self.mu, prev_h, fb.seq_cu,
                                    fb.seq_start, fb.seq_slots, fb.row_seq)
        rkvg = torch.bmm(mixes[:4], self.rkvg_t)          # [4, T, H*N]
        lw = F.linear(torch.tanh(F.linear(mixes[4].float(), self.w1)),
                      self.w2, self.w0)                    # fp32 [T, H*N]
        o, _ = ops.outer_scan(
            rkvg[0].view(T, H, N), rkvg[1].view(T, H, N),
            rkvg[2].view(T, H, N), lw.view(T, H, N), None, self.bonus, None,
            mem, fb.seq_cu, fb.seq_start, fb.seq_slots, fb.seq_rows,
            ops.DECAY_EXP_NEG_EXP, False, 1.0)
        y = ops.head_norm_gate(o, rkvg[3], self.norm_w, self.eps, N,
                               ops.GATE_SILU, False, None, None, self.dtype)
        return F.linear(y, self.o)


class ParallelMixer(nn.Module):
    """Two mixers read the same input; each output is RMS-normed over
    the model width with its own plain weight, and the two are averaged.
    `left` and `right` are any two mixer modules whose cache_spec() is a
    list of buffers and whose forward is (h, batch, buffers)."""

    def __init__(self, hidden: int, left: nn.Module, right: nn.Module,
                 eps: float, name: str, device):
        super().__init__()
        self.eps = eps
        self.left, self.right = left, right
        self.n_left = len(left.cache_spec())
        self.left_out = _param(1.0 + _rand((hidden,), device, torch.float32,
                                           name + ".left.out", 5.0))
        self.right_out = _param(1.0 + _rand((hidden,), device,
                                            torch.float32,
                                            name + ".right.out", 5.0))

    def cache_spec(self):
        return ("group", self.left.cache_spec() + self.right.cache_spec())

    def forward(self, h, fb: ForwardBatch, cache):
        a = self.left(h, fb, cache[:self.n_left])
        b = self.right(h, fb, cache[self.n_left:])
        return ops.rmsnorm_pair_mean(a, b, self.left_out, self.right_out,
                                     self.eps)


class Relu2MLP(nn.Module):
    """W_down relu(W_up h)^2."""

    def __init__(self, hidden: int, ff: int, name: str, device, dtype):
        super().__init__()
        self.up = _w((ff, hidden), device, dtype, name + ".up", hidden)
        self.down = _w((hidden, ff), device, dtype, name + ".down", ff)

    def forward(self, h):
        return F.linear(ops.relu2(F.linear(h, self.up)), self.down)


class FeditarLayer(nn.Module):
    def __init__(self, cfg: FeditarConfig, i: int, device, dtype):
        super().__init__()
        spec = cfg.layers[i]
        D, eps = cfg.hidden_size, cfg.norm_eps
        self.eps, self.dtype = eps, dtype
        self.norm1_w = _one_plus(D, device, f"l{i}.norm1")
        name = f"l{i}.mix"
        if spec.type == "mlstm":
            self.mixer = MLSTMMixer(D, spec.mixer, eps, name, device, dtype)
        elif spec.type == "mamba2":
            self.mixer = Mamba2Mixer(D, spec.mixer, eps, name, device, dtype)
        elif spec.type == "parallel":
            self.mixer = ParallelMixer(
                D, SoftcapAttention(D, spec.mixer.left, name + ".left",
                                    device, dtype),
                DecayMemory(D, spec.mixer.right, eps, name + ".right",
                            device, dtype), eps, name, device)
        else:
            raise ValueError(f"layer {i}: unknown mixer {spec.type!r}")
        if spec.mlp is None:
            self.norm2_w = self.mlp = None
        else:
            self.norm2_w = _one_plus(D, device, f"l{i}.norm2")
            self.mlp = Relu2MLP(D, spec.mlp.ff, f"l{i}.mlp", device, dtype)

    def forward(self, residual, delta, fb, cache):
        """residual: fp32 stream, updated in place with the PREVIOUS
        sub-block's output `delta` inside the fused add + norm; returns
        this layer's last un-added output."""
        h, _ = ops.add_rmsnorm_pair(residual, delta, None, self.norm1_w,
                                    None, self.eps, self.dtype)
        delta = self.mixer(h, fb, cache)
        if self.mlp is not None:
            h, _ = ops.add_rmsnorm_pair(residual, delta, None, self.norm2_w,
                                        None, self.eps, self.dtype)
            delta = self.mlp(h)
        return delta


class FeditarForCausalLM(nn.Module):
    needs_seq_meta = True          # ForwardBatch.seq_* / row_seq fields
    supports_decode_graph = False  # decode runs eagerly
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, cfg: FeditarConfig, device, dtype=torch.bfloat16):
        super().__init__()
        if tp_world_size() != 1:
            raise ValueError("Feditar runs unsharded (tensor parallel "
                             "degree 1)")
        self.cfg = cfg
        self.device = device
        self.dtype = dtype
        D = cfg.hidden_size
        self.embed = _param(_rand((cfg.vocab_size, D), device, dtype,
                                  "embed", 50.0 / cfg.embed_scale))
        self.pair = _param(_rand((cfg.pair_hash.buckets + 1, D), device,
                                 dtype, "bigram", 25.0))
        self.pos = _param(_rand((cfg.max_position, D), device, dtype, "pos",
                                25.0))
        self.embed_norm_w = _one_plus(D, device, "embed.norm")
        self.layers = nn.ModuleList(
            FeditarLayer(cfg, i, device, dtype)
            for i in range(cfg.num_layers))
        self.final_norm_w = _one_plus(D, device, "final.norm")
        self.tap = None    # debugging hook: called with (layer, residual)
        # the engine caps its sequence length at the learned table
        self.position_table_rows = cfg.max_position

    def cache_specs(self) -> List[tuple]:
        """One entry per layer (a group of slot buffers, plus paged K/V
        for a parallel mixer) and a last one for the embedding: each
        sequence's previous token."""
        return [l.mixer.cache_spec() for l in self.layers] + [
            ("slot_i32", 1)]

    def forward(self, fb: ForwardBatch, caches) -> torch.Tensor:
        cfg = self.cfg
        ph = cfg.pair_hash
        residual = ops.embed_pair_norm(
            fb.token_ids, fb.positions, caches[len(self.layers)], fb.seq_cu,
            fb.seq_start, fb.seq_slots, fb.row_seq, self.embed, self.pair,
            self.pos, self.embed_norm_w, cfg.embed_scale, ph.buckets,
            ph.mul_prev, ph.mul_cur, cfg.norm_eps)
        delta = None
        for i, layer in enumerate(self.layers):
            delta = layer(residual, delta, fb, caches[i])
            if self.tap is not None:
                self.tap(i, residual + delta.float())
        h, _ = ops.add_rmsnorm_pair(residual, delta, None, self.final_norm_w,
                                    None, cfg.norm_eps, self.dtype)
        return h

    def compute_logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.embed).float()
