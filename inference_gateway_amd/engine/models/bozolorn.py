"""Bozolorn: a per-layer decoder with sandwich norms for the MI355X engine.

The fp32 residual stream starts as the scaled token row.  Every sublayer
is normed on the way in AND on the way out,

    x <- x + norm1b(mixer(norm1 x));   x <- x + norm2b(ff(norm2 x))

and after the feed-forward every layer adds a small function of the token
itself: a slice of a second, narrow embedding table, gated by the residual
(TokenSideInput).  Mixers, chosen per layer:

  ChunkBiasAttention   softmax attention without rotation; a linear bias
                       per head on the distance, keys only from the row's
                       own chunk of positions, sigmoid output gate; a
                       layer may read ANOTHER layer's paged keys and
                       values instead of projecting its own
  ParallelMixer        SinkRotaryAttention (projection biases, per-head
                       q/k RMS norm, partial interleaved rotary positions
                       with YaRN interpolation, a unit sink in the softmax
                       denominator) beside GatedDeltaMixer (short
                       convolutions + silu on q/k/v, unit-length q/k, a
                       decayed memory corrected by the delta rule, gated
                       per-head norm); the two outputs are normed over the
                       width and averaged (engine/models/feditar.py)

The feed-forward is GroupRoutedMoE: clamped gated experts behind a sigmoid
router that chooses inside the best expert groups.

Everything a layer keeps between steps is paged K/V or a slot buffer
handed in by the engine (cache_specs), so portions of prompts, decoded
tokens and mixed batches are one code path.  GEMMs go through
F.linear/bmm; the small projections that feed the recurrence's gates and
the router run in fp32; everything between GEMMs is a gfx950 kernel from
ops.
"""
from __future__ import annotations

from typing import List

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import ops
from ...parallel.comm import tp_world_size
from ..config import (BozolornConfig, ChunkBiasAttentionSpec, DeltaRuleSpec,
                      GroupRoutedSpec, SinkAttentionSpec)
from . import moe_common
from .batch import ForwardBatch
from .fedatar import _param, _rand
from .feditar import ParallelMixer


def _w(shape, device, dtype, name, fan_in):
    return _param(_rand(shape, device, dtype, name, fan_in ** -0.5 / 0.02))


def _norm_w(n, device, name):
    return _param(1.0 + _rand((n,), device, torch.float32, name, 5.0))


class ChunkBiasAttention(nn.Module):
    """score(i, j) = q_i . k_j * scale - slope_h (i - j), slope_h =
    2^(-8 (h + 1) / H); j <= i and floor(j / chunk) = floor(i / chunk);
    softmax; heads concatenated, times sigmoid(W_g h), then W_o.  With
    spec.kv_from >= 0 the layer has no key/value projections and reads
    the cache of that layer."""

    def __init__(self, hidden: int, spec: ChunkBiasAttentionSpec, name: str,
                 device, dtype):
        super().__init__()
        self.spec = spec
        H, G, N, P = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        self.owns_kv = spec.kv_from < 0
        self.nq = H * N
        self.nk, self.nv = (G * N, G * P) if self.owns_kv else (0, 0)
        # fused projection rows: q | k | v (own keys/values only) | gate
        self.qkvg = _w((self.nq + self.nk + self.nv + H * P, hidden),
                       device, dtype, name + ".qkvg", hidden)
        self.o = _w((hidden, H * P), device, dtype, name + ".o", H * P)
        self.register_buffer("slopes", torch.tensor(
            [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
            dtype=torch.float32, device=device), persistent=False)

    def cache_spec(self):
        s = self.spec
        if not self.owns_kv:
            return ("group", [])
        return ("paged_k_v", s.kv_heads, s.dim, s.vdim)

    def forward(self, h, fb: ForwardBatch, cache):
        """cache: this layer's (K, V) pages, or its source layer's."""
        kc, vc = cache
        s = self.spec
        proj = F.linear(h, self.qkvg)
        k0, v0 = self.nq, self.nq + self.nk
        if self.owns_kv:
            ops.append_paged_kv(proj[:, k0:v0], proj[:, v0:v0 + self.nv],
                                kc, vc, fb.slot_mapping)
        o = ops.softcap_attention(
            proj[:, :self.nq], kc, vc, fb.seq_block_table, fb.row_seq,
            fb.positions, s.scale, 0.0, 0.0, 1, 0, fb.num_chunk_rows,
            fb.seq_lens, fb.seq_cu, fb.seq_start, slopes=self.slopes,
            chunk=s.chunk, gate=proj[:, v0 + self.nv:])
        return F.linear(o, self.o)


class SinkRotaryAttention(nn.Module):
    """q, k, v = W h + b; q and k RMS-normed per head (one weight vector
    shared by the heads) and rotated on their first rot.dims entries;
    causal; p_j = exp(s_j) / (1 + sum exp(s)); W_o."""

    def __init__(self, hidden: int, spec: SinkAttentionSpec, eps: float,
                 name: str, device, dtype):
        super().__init__()
        self.spec, self.eps = spec, eps
        H, G, N, P = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        rows = H * N + G * N + G * P
        self.qkv = _w((rows, hidden), device, dtype, name + ".qkv", hidden)
        self.qkv_b = _param(_rand((rows,), device, dtype, name + ".qkv_b",
                                  10.0))
        self.qnorm_w = _norm_w(N, device, name + ".q.norm")
        self.knorm_w = _norm_w(N, device, name + ".k.norm")
        self.o = _w((hidden, H * P), device, dtype, name + ".o", H * P)
        self.mag = 1.0
        if spec.rot is not None and spec.rot.dims > 0:
            freq, self.mag = spec.rot.frequencies()
            self.register_buffer("inv_freq", torch.tensor(
                freq, dtype=torch.float64).to(torch.float32).to(device),
                persistent=False)
        else:
            self.inv_freq = None
        # the sink: one more softmax term of score 0 for every head
        self.register_buffer("sinks", torch.zeros(
            H, dtype=torch.float32, device=device), persistent=False)

    def cache_spec(self):
        s = self.spec
        return [("paged_k_v", s.kv_heads, s.dim, s.vdim)]

    def forward(self, h, fb: ForwardBatch, cache):
        (kc, vc), = cache
        s = self.spec
        proj = F.linear(h, self.qkv, self.qkv_b)
        q = ops.qk_norm_rope_append(
            proj, fb.positions, fb.slot_mapping, kc, vc, self.qnorm_w,
            self.knorm_w, self.inv_freq, self.mag, self.eps, s.heads,
            s.kv_heads, s.dim, s.vdim)
        o = ops.softcap_attention(
            q, kc, vc, fb.seq_block_table, fb.row_seq, fb.positions,
            s.scale, 0.0, 0.0, 1, 0, fb.num_chunk_rows, fb.seq_lens,
            fb.seq_cu, fb.seq_start, sinks=self.sinks)
        return F.linear(o, self.o)


class GatedDeltaMixer(nn.Module):
    """q, k (kv_heads x dim) and v (heads x vdim) pass a short causal
    convolution and silu; q and k are scaled to unit length per head (q
    also by dim^-1/2); per head: S <- a S, u = b (v - S^T k), S <- S + k
    u^T, o = S^T q with a = exp(-exp(A_log) softplus(W_a h + dt_bias)),
    b = sigmoid(W_b h); o RMS-normed per head, times silu(W_g h), W_o."""

    UNIT_EPS = 1e-6

    def __init__(self, hidden: int, spec: DeltaRuleSpec, eps: float,
                 name: str, device, dtype):
        super().__init__()
        self.spec, self.eps, self.dtype = spec, eps, dtype
        H, P = spec.heads, spec.vdim
        CC = spec.conv_channels
        # fused projection rows: q | k | v | output-gate logits
        self.qkvg = _w((CC + H * P, hidden), device, dtype, name + ".qkvg",
                       hidden)
        self.conv_w = _param(_rand((CC, spec.conv), device, torch.float32,
                                   name + ".conv", 25.0))
        # step | write-strength logits, fp32
        self.ab_w = _w((2 * H, hidden), device, torch.float32, name + ".ab",
                       hidden)
        self.a_log = _param(_rand((H,), device, torch.float32,
                                  name + ".A_log", 25.0))
        self.dt_bias = _param(_rand((H,), device, torch.float32,
                                    name + ".dt_bias", 25.0))
        # the per-head norm weight, repeated for every head
        self.norm_w = _norm_w(H * P, device, name + ".norm")
        self.o = _w((hidden, H * P), device, dtype, name + ".o", H * P)

    def cache_spec(self):
        s = self.spec
        return [("state", max(1, (s.conv - 1) * s.conv_channels)),
                ("state", s.heads * s.dim * s.vdim)]

    def forward(self, h, fb: ForwardBatch, cache):
        conv_state, mem = cache
        s = self.spec
        H, G, N, P = s.heads, s.kv_heads, s.dim, s.vdim
        T, GN, CC = h.shape[0], G * N, s.conv_channels
        proj = F.linear(h, self.qkvg)
        decay, beta = ops.decay_beta_gates(
            F.linear(h.float(), self.ab_w), self.a_log, self.dt_bias)
        c = ops.causal_conv(proj[:, :CC], self.conv_w, None, conv_state,
                            fb.seq_cu, fb.seq_start, fb.seq_slots,
                            fb.row_seq, True)
        o = ops.delta_scan(
            c[:, :GN].view(T, G, N), c[:, GN:2 * GN].view(T, G, N),
            c[:, 2 * GN:].view(T, H, P), decay, beta, mem, fb.seq_cu,
            fb.seq_start, fb.seq_slots, fb.seq_rows, self.UNIT_EPS,
            float(N) ** -0.5)
        y = ops.head_norm_gate(o, proj[:, CC:], self.norm_w, self.eps, P,
                               ops.GATE_SILU, False, None, None, self.dtype)
        return F.linear(y, self.o)


class GroupRoutedMoE(nn.Module):
    """Router scores s = sigmoid(W_r h) in fp32; experts are chosen by s
    + correction inside the best expert groups (ops.moe_group_route) and
    weighted by s, not renormalised.  Expert: W_down (g' sigmoid(ALPHA
    g') (u' + 1)), g' = min(W_gate h, L), u' = clamp(W_up h, -L, L).
    Expert weights are stored K-major ([E, in, out]) for the batched
    GEMMs, gate and up stacked."""

    ALPHA = 1.702
    PADDED_MAX_ROWS = 256

    def __init__(self, hidden: int, spec: GroupRoutedSpec, name: str, device,
                 dtype):
        super().__init__()
        self.spec = spec
        E, f = spec.experts, spec.expert_ff
        self.router_w = _w((E, hidden), device, torch.float32,
                           name + ".router", hidden)
        self.correction = _param(_rand((E,), device, torch.float32,
                                       name + ".correction", 5.0))
        self.up_t = _w((E, hidden, 2 * f), device, dtype, name + ".up",
                       hidden)
        self.down_t = _w((E, f, hidden), device, dtype, name + ".down", f)

    def _act(self, z: torch.Tensor) -> torch.Tensor:
        return ops.gated_act(z, ops.GATED_ACT_CLAMPED, self.spec.limit,
                             self.ALPHA)

    def forward(self, h: torch.Tensor, fb: ForwardBatch) -> torch.Tensor:
        sp = self.spec
        T = h.shape[0]
        logits = F.linear(h.float(), self.router_w)
        padded = T <= self.PADDED_MAX_ROWS
        C = (T + 63) // 64 * 64
        weights, idx, dst = ops.moe_group_route(
            logits, self.correction, sp.top, sp.groups, sp.keep,
            C if padded else 0)
        if padded:
            if dst is None:
                dst = moe_common.padded_rows(idx, sp.experts, C)
            return moe_common.experts_padded(h, weights, dst, self.up_t,
                                             self.down_t, C, self._act)
        return moe_common.experts_sorted(h, weights, idx, self.up_t,
                                         self.down_t, self._act)


class TokenSideInput(nn.Module):
    """y = W_proj (gelu_tanh(W_gate x) * e), e = this layer's slice of
    the token's row in the shared narrow table; the layer adds rmsnorm(y)
    * norm_w to the stream."""

    def __init__(self, hidden: int, dim: int, index: int, name: str, device,
                 dtype):
        super().__init__()
        self.col0 = index * dim
        self.gate = _w((dim, hidden), device, dtype, name + ".gate", hidden)
        self.proj = _w((hidden, dim), device, dtype, name + ".proj", dim)
        self.norm_w = _norm_w(hidden, device, name + ".norm")

    def forward(self, x, table, token_ids):
        g = ops.gelu_mul_rows(F.linear(x, self.gate), table, token_ids,
                              self.col0)
        return F.linear(g, self.proj)


class BozolornLayer(nn.Module):
    def __init__(self, cfg: BozolornConfig, i: int, device, dtype):
        super().__init__()
        spec = cfg.layers[i]
        D, eps = cfg.hidden_size, cfg.norm_eps
        self.eps, self.dtype = eps, dtype
        self.norm1_w = _norm_w(D, device, f"l{i}.norm1")
        self.norm1b_w = _norm_w(D, device, f"l{i}.norm1b")
        name = f"l{i}.mix"
        self.kv_from = -1
        if spec.type == "attention":
            self.mixer = ChunkBiasAttention(D, spec.mixer, name, device,
                                            dtype)
            self.kv_from = spec.mixer.kv_from
        elif spec.type == "parallel":
            self.mixer = ParallelMixer(
                D, SinkRotaryAttention(D, spec.mixer.left, eps,
                                       name + ".left", device, dtype),
                GatedDeltaMixer(D, spec.mixer.right, eps, name + ".right",
                                device, dtype), eps, name, device)
        else:
            raise ValueError(f"layer {i}: unknown mixer {spec.type!r}")
        if spec.mlp is None:
            self.norm2_w = self.norm2b_w = self.mlp = None
        else:
            self.norm2_w = _norm_w(D, device, f"l{i}.norm2")
            self.norm2b_w = _norm_w(D, device, f"l{i}.norm2b")
            self.mlp = GroupRoutedMoE(D, spec.mlp, f"l{i}.mlp", device,
                                      dtype)
        self.side = TokenSideInput(D, cfg.side_dim, i, f"l{i}.side", device,
                                   dtype) if cfg.side_dim else None

    def forward(self, residual, delta, w_post, fb, cache, side_table):
        """residual: fp32 stream; (delta, w_post): the PREVIOUS
        sublayer's output and the weight of its outgoing norm, added
        inside this layer's first fused norm kernel.  Returns this
        layer's last un-added pair."""
        h = ops.add_normed_rmsnorm(residual, delta, w_post, self.norm1_w,
                                   self.eps, self.dtype)
        delta, w_post = self.mixer(h, fb, cache), self.norm1b_w
        if self.mlp is not None:
            h = ops.add_normed_rmsnorm(residual, delta, w_post,
                                       self.norm2_w, self.eps, self.dtype)
            delta, w_post = self.mlp(h, fb), self.norm2b_w
        if self.side is not None:
            x = ops.add_normed_rmsnorm(residual, delta, w_post, None,
                                       self.eps, self.dtype)
            delta = self.side(x, side_table, fb.token_ids)
            w_post = self.side.norm_w
        return delta, w_post


class BozolornForCausalLM(nn.Module):
    needs_seq_meta = True          # ForwardBatch.seq_* / row_seq fields
    supports_decode_graph = False  # decode runs eagerly
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, cfg: BozolornConfig, device, dtype=torch.bfloat16):
        super().__init__()
        if tp_world_size() != 1:
            raise ValueError("Bozolorn runs unsharded (tensor parallel "
                             "degree 1)")
        self.cfg = cfg
        self.device = device
        self.dtype = dtype
        D = cfg.hidden_size
        self.embed = _param(_rand((cfg.vocab_size, D), device, dtype,
                                  "embed", 50.0 / cfg.embed_scale))
        self.side_embed = _param(_rand(
            (cfg.vocab_size, cfg.side_dim * cfg.num_layers), device, dtype,
            "side.embed", 50.0)) if cfg.side_dim else None
        self.layers = nn.ModuleList(
            BozolornLayer(cfg, i, device, dtype)
            for i in range(cfg.num_layers))
        self.final_norm_w = _norm_w(D, device, "final.norm")
        self.head = _w((cfg.vocab_size, D), device, dtype, "head", D)
        self.tap = None    # debugging hook: called with (layer, residual)

    def cache_specs(self) -> List[tuple]:
        """One entry per layer: paged K/V for an attention layer that
        projects its own (nothing for one that borrows), paged K/V plus
        the delta-rule memory and its filter history for a parallel
        layer."""
        return [l.mixer.cache_spec() for l in self.layers]

    def forward(self, fb: ForwardBatch, caches) -> torch.Tensor:
        cfg = self.cfg
        residual = F.embedding(fb.token_ids, self.embed).float()
        if cfg.embed_scale != 1.0:
            residual.mul_(cfg.embed_scale)
        delta = w_post = None
        for i, layer in enumerate(self.layers):
            cache = caches[layer.kv_from if layer.kv_from >= 0 else i]
            delta, w_post = layer(residual, delta, w_post, fb, cache,
                                  self.side_embed)
            if self.tap is not None:
                d = delta.float()
                self.tap(i, residual + d * torch.rsqrt(
                    (d * d).mean(-1, keepdim=True) + cfg.norm_eps) * w_post)
        return ops.add_normed_rmsnorm(residual, delta, w_post,
                                      self.final_norm_w, cfg.norm_eps,
                                      self.dtype)

    def compute_logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.head).float()
