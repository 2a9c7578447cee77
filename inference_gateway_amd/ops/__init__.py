"""Op dispatch for the MI355X engine.

On a GPU box the hand-written gfx950 HIP kernels (_kernels extension) are
REQUIRED — if a CUDA/HIP device is visible and the extension is missing,
every op raises instead of silently falling back to eager PyTorch (the
round-end harness records which .so files the GPU processes load). On CPU
the fp32 torch references (torch_ref) run so the whole engine and gateway
are testable without a GPU.
"""
from __future__ import annotations

import torch

from . import torch_ref

try:
    from . import _kernels  # compiled by setup.py build_ext --inplace

    HAS_KERNELS = True
except ImportError:  # pragma: no cover - absent only before first build
    _kernels = None
    HAS_KERNELS = False


try:
    from . import _hybrid  # recurrent / latent-attention mechanisms

    HAS_HYBRID = True
except ImportError:  # pragma: no cover - absent only before first build
    _hybrid = None
    HAS_HYBRID = False


try:
    from . import _recurrent  # matrix-memory / state-space / decay mixers

    HAS_RECURRENT = True
except ImportError:  # pragma: no cover - absent only before first build
    _recurrent = None
    HAS_RECURRENT = False


def _require_recurrent() -> None:
    if not HAS_RECURRENT:
        raise RuntimeError(
            "inference_gateway_amd.ops._recurrent is not built but a GPU "
            "tensor was passed. Build it in-tree with: "
            "IGW_BUILD_EXT=recurrent PYTORCH_ROCM_ARCH=gfx950 python "
            "setup.py build_ext --inplace"
        )


def _shared_ext(name: str):
    """The row-wise ops that both the hybrid and the recurrent extension
    compile (same source file): whichever is loaded serves them, so a
    process that runs one model family loads one library."""
    for ext in (_hybrid, _recurrent):
        if ext is not None and hasattr(ext, name):
            return getattr(ext, name)
    _require_hybrid()


def _require_hybrid() -> None:
    if not HAS_HYBRID:
        raise RuntimeError(
            "inference_gateway_amd.ops._hybrid is not built but a GPU "
            "tensor was passed. Build it in-tree with: IGW_BUILD_EXT=hybrid "
            "PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace"
        )


def _require_kernels() -> None:
    if not HAS_KERNELS:
        raise RuntimeError(
            "inference_gateway_amd.ops._kernels is not built but a GPU tensor "
            "was passed. Build it in-tree with: "
            "PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace"
        )


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        _require_kernels()
        out = torch.empty_like(x)
        _kernels.rmsnorm(out, x, weight, eps)
        return out
    return torch_ref.rmsnorm_ref(x, weight, eps)


def fused_add_rmsnorm(x, residual, weight, eps: float):
    """In-place: residual += x; x = rmsnorm(residual) * w. Returns (x, residual)."""
    if x.is_cuda:
        _require_kernels()
        _kernels.fused_add_rmsnorm(x, residual, weight, eps)
        return x, residual
    nx, nres = torch_ref.fused_add_rmsnorm_ref(x, residual, weight, eps)
    x.copy_(nx)
    residual.copy_(nres)
    return x, residual


def rotary_embedding(positions, q, k, head_dim: int, cos_sin_cache):
    """In-place NeoX RoPE on q [T, NQ*HD] and k [T, NKV*HD]."""
    if q.is_cuda:
        _require_kernels()
        _kernels.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)
        return q, k
    nq, nk = torch_ref.rope_ref(positions, q, k, head_dim, cos_sin_cache)
    q.copy_(nq)
    k.copy_(nk)
    return q, k


def append_kv_cache(k, v, kcache, vcache, slot_mapping):
    if k.is_cuda:
        _require_kernels()
        _kernels.append_kv_cache(k, v, kcache, vcache, slot_mapping)
        return
    torch_ref.append_kv_cache_ref(k, v, kcache, vcache, slot_mapping)


def paged_attn_decode(q, kcache, vcache, block_table, ctx_lens, scale: float):
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        _kernels.paged_attn_decode(
            out, q, kcache, vcache, block_table, ctx_lens, scale
        )
        return out
    return torch_ref.paged_attn_decode_ref(
        q, kcache, vcache, block_table, ctx_lens, scale
    )


def flash_prefill(q, k, v, cu_seqlens, seq_lens, scale: float):
    """Varlen causal prefill attention. seq_lens: python list of ints."""
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        tile_seq, tile_off = torch_ref.make_prefill_tiles(
            seq_lens, tile_m=64, device=q.device
        )
        _kernels.flash_prefill(
            out, q, k, v, cu_seqlens, tile_seq, tile_off, scale
        )
        return out
    return torch_ref.flash_prefill_ref(q, k, v, cu_seqlens, scale)


def flash_prefill_paged(q, kcache, vcache, block_table, prefix_lens,
                        cu_seqlens, seq_lens, scale: float):
    """Paged-EXTEND prefill (chunked-prefill / prefix-cache enabler):
    q rows are a per-seq CHUNK whose own K/V plus `prefix_lens` cached
    tokens before it are all in the paged cache; each q row attends over
    cache positions [0, prefix + row].  seq_lens: python ints (q rows
    per sequence)."""
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        tile_seq, tile_off = torch_ref.make_prefill_tiles(
            seq_lens, tile_m=64, device=q.device
        )
        _kernels.flash_prefill_paged(
            out, q, kcache, vcache, block_table, prefix_lens, cu_seqlens,
            tile_seq, tile_off, scale
        )
        return out
    return torch_ref.flash_prefill_paged_ref(
        q, kcache, vcache, block_table, prefix_lens, cu_seqlens, scale
    )


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    if gate_up.is_cuda:
        _require_kernels()
        inter = gate_up.shape[-1] // 2
        out = torch.empty(
            (*gate_up.shape[:-1], inter),
            dtype=gate_up.dtype,
            device=gate_up.device,
        )
        _kernels.silu_mul(out, gate_up)
        return out
    return torch_ref.silu_mul_ref(gate_up)


def sample(logits, temperature, top_k, top_p, uniforms):
    """logits [B, V] fp32 -> sampled token ids [B] int32."""
    if logits.is_cuda:
        _require_kernels()
        out = torch.empty(
            logits.shape[0], dtype=torch.int32, device=logits.device
        )
        _kernels.sample(out, logits, temperature, top_k, top_p, uniforms)
        return out
    return torch_ref.sample_ref(logits, temperature, top_k, top_p, uniforms)


build_cos_sin_cache = torch_ref.build_cos_sin_cache
rotary_inv_freq = torch_ref.rotary_inv_freq
make_prefill_tiles = torch_ref.make_prefill_tiles


def moe_route(router_logits: torch.Tensor, top_k: int, capacity: int):
    """Fused MoE routing: top-k + softmax + padded-dispatch row indices.

    router_logits: [T, E] fp32. Returns (weights [T,K] fp32,
    dst [T*K] int32, topk_idx [T,K] int32, counts [E] int32)."""
    if router_logits.is_cuda:
        _require_kernels()
        T, E = router_logits.shape
        weights = torch.empty((T, top_k), dtype=torch.float32,
                              device=router_logits.device)
        dst = torch.empty(T * top_k, dtype=torch.int32,
                          device=router_logits.device)
        topk_idx = torch.empty((T, top_k), dtype=torch.int32,
                               device=router_logits.device)
        counts = torch.empty(E, dtype=torch.int32,
                             device=router_logits.device)
        _kernels.moe_route(weights, dst, topk_idx, counts, router_logits,
                           capacity)
        return weights, dst, topk_idx, counts
    return torch_ref.moe_route_ref(router_logits, top_k, capacity)


def moe_grouped_gemm(a: torch.Tensor, w: torch.Tensor,
                     counts: torch.Tensor, capacity: int) -> torch.Tensor:
    """Per-expert GEMM over the padded dispatch buffer.

    a: [E*C, K] bf16 (rows >= counts[e] in each expert segment are
    ignored), w: [E, N, K] bf16 -> out [E*C, N] bf16 (only real rows
    written)."""
    if a.is_cuda:
        _require_kernels()
        E, N, _K = w.shape
        out = torch.empty((a.shape[0], N), dtype=a.dtype, device=a.device)
        _kernels.moe_grouped_gemm(out, a, w, counts, capacity)
        return out
    return torch_ref.moe_grouped_gemm_ref(a, w, counts, capacity)


def silu_mul_grouped(gate_up: torch.Tensor, counts: torch.Tensor,
                     capacity: int) -> torch.Tensor:
    """SwiGLU over only the real rows of the padded dispatch buffer."""
    if gate_up.is_cuda:
        _require_kernels()
        inter = gate_up.shape[-1] // 2
        out = torch.empty((*gate_up.shape[:-1], inter), dtype=gate_up.dtype,
                          device=gate_up.device)
        _kernels.silu_mul_grouped(out, gate_up, counts, capacity)
        return out
    return torch_ref.silu_mul_grouped_ref(gate_up, counts, capacity)


def fused_gemm_tn(x: torch.Tensor, w: torch.Tensor, swiglu: bool = False,
                  nt_weights: bool = False) -> torch.Tensor:
    """TN bf16 GEMM out = x @ w.T with an optional fused SwiGLU
    epilogue (w = [gate; up] rows, out = silu(g)*u).  Decode
    weight-streaming shapes (M%128==0, N%64==0, K%32==0); callers fall
    back to the library GEMM otherwise (ops/csrc/fused_gemm.hip)."""
    if x.is_cuda:
        _require_kernels()
        N = w.shape[0] // 2 if swiglu else w.shape[0]
        out = torch.empty((x.shape[0], N), dtype=x.dtype, device=x.device)
        _kernels.fused_gemm_tn(out, x, w, swiglu, nt_weights)
        return out
    y = x.float() @ w.float().t()
    if swiglu:
        N = w.shape[0] // 2
        g, u = y[:, :N], y[:, N:]
        y = torch.nn.functional.silu(g) * u
    return y.to(x.dtype)


def fused_gemm_tn_supported(M: int, N_rows: int, K: int,
                            swiglu: bool) -> bool:
    N = N_rows // 2 if swiglu else N_rows
    return M % 128 == 0 and N % 64 == 0 and K % 32 == 0


# ---------------------------------------------------------------------------
# Hybrid-decoder mechanisms: fp32-residual LayerNorm, minGRU scan, windowed
# latent attention with a softmax sink, xIELU / relu^2 activations.  The
# kernels are typed for bf16 AND fp32 activations (true 32-bit serving);
# norms, recurrent state, angles and softmax are fp32 in both.
# ---------------------------------------------------------------------------
def add_layernorm(residual, delta, weight, bias, eps: float, out_dtype):
    """residual [T, D] fp32 += delta (in place; delta may be None);
    returns LayerNorm(residual) * weight + bias in out_dtype."""
    if residual.is_cuda:
        _require_hybrid()
        out = torch.empty(residual.shape, dtype=out_dtype,
                          device=residual.device)
        _hybrid.add_layernorm(out, residual, delta, weight, bias, eps)
        return out
    return torch_ref.add_layernorm_ref(residual, delta, weight, bias, eps,
                                       out_dtype)


# rows per chunk of the chunked minGRU scan, and the segment length from
# which it replaces the one-thread-per-channel walk
MINGRU_CHUNK = 16
MINGRU_CHUNKED_FROM = 256


def mingru_scan(zug, state, seq_cu, seq_start, seq_slots, seq_rows):
    """minGRU recurrence + output gate over a ragged batch.  zug [T, 3W]
    (z | x | g pre-activations), state [slots, W] fp32 (read when the
    sequence's first row is not position 0, always written back).
    seq_rows: python row counts per sequence (host side; picks the
    sequential or the chunked-scan schedule and lays out its chunks)."""
    if zug.is_cuda:
        _require_hybrid()
        W = zug.shape[1] // 3
        out = torch.empty((zug.shape[0], W), dtype=zug.dtype,
                          device=zug.device)
        if max(seq_rows) < MINGRU_CHUNKED_FROM:
            _hybrid.mingru_scan(out, zug, state, seq_cu, seq_start,
                                seq_slots)
            return out
        tab, ccu_t = _scan_chunks(tuple(seq_rows), MINGRU_CHUNK, zug.device)
        work = torch.empty((2, tab.shape[1], W), dtype=torch.float32,
                           device=zug.device)
        _hybrid.mingru_scan_chunked(out, zug, state, seq_start, seq_slots,
                                    tab[0], tab[1], ccu_t, work)
        return out
    return torch_ref.mingru_scan_ref(zug, state, seq_cu, seq_start,
                                     seq_slots)


def rope_pairs_(x, positions, inv_freq, offset: int):
    """In-place interleaved-pair rotation of x[T, H, hd][..., offset :
    offset + 2*len(inv_freq)] by positions * inv_freq (fp32 angles)."""
    if x.is_cuda:
        _require_hybrid()
        _hybrid.rope_pairs(x, positions, inv_freq, offset)
        return x
    return torch_ref.rope_pairs_ref(x, positions, inv_freq, offset)


def latent_down_post(down, positions, slot_mapping, cache, qnorm_w,
                     kvnorm_w, inv_freq, eps: float, q_rank: int,
                     kv_rank: int, rot_dim: int, heads: int):
    """Post-processing of the fused down projection [T, q_rank + kv_rank
    + rot_dim + heads]: returns (normed query latent [T, q_rank],
    sigmoid head gates [T, heads] fp32) and appends (normed latent |
    rotated shared key) to the paged cache at slot_mapping."""
    if down.is_cuda:
        _require_hybrid()
        T = down.shape[0]
        cq = torch.empty((T, q_rank), dtype=down.dtype, device=down.device)
        gate = torch.empty((T, heads), dtype=torch.float32,
                           device=down.device)
        _hybrid.latent_down_post(cq, gate, down, positions, slot_mapping,
                                  cache, qnorm_w, kvnorm_w, inv_freq, eps,
                                  q_rank, kv_rank, rot_dim, heads)
        return cq, gate
    return torch_ref.latent_down_post_ref(
        down, positions, slot_mapping, cache, qnorm_w, kvnorm_w, inv_freq,
        eps, q_rank, kv_rank, rot_dim, heads)


import functools


@functools.lru_cache(maxsize=256)
def _attention_tiles(tq: int, num_prefill_rows: int, seq_lens: tuple,
                     T: int, device):
    """[2, ntiles] int32 (first row, row count) of the attention tiles:
    prompt portions cut into runs of tq rows, decoded rows one each.
    Cached: serving repeats the same batch shapes."""
    row0, nrows, row = [], [], 0
    for n in seq_lens:
        for a in range(0, n, tq):
            row0.append(row + a)
            nrows.append(min(tq, n - a))
        row += n
    assert row == num_prefill_rows
    row0.extend(range(num_prefill_rows, T))
    nrows.extend([1] * (T - num_prefill_rows))
    return torch.tensor([row0, nrows], dtype=torch.int32).to(device)


@functools.lru_cache(maxsize=256)
def _scan_chunks(seq_rows: tuple, chunk: int, device):
    """Chunk table of the chunked minGRU scan: ([2, NC] row ranges,
    [S+1] chunk offsets per sequence), cached per batch shape."""
    r0, r1, ccu, row = [], [], [0], 0
    for n in seq_rows:
        for a in range(0, n, chunk):
            r0.append(row + a)
            r1.append(row + min(n, a + chunk))
        row += n
        ccu.append(len(r0))
    return (torch.tensor([r0, r1], dtype=torch.int32).to(device),
            torch.tensor(ccu, dtype=torch.int32).to(device))


# bf16 batches run the MFMA tile kernel; off = the one-wave-per-row kernel
# (any dtype, any sizes) for everything
LATENT_ATTENTION_MFMA = True


def latent_attention(q_abs, q_rot, cache, block_table, row_seq, positions,
                     sink, scale: float, window: int,
                     num_prefill_rows: int = 0, prefill_seq_lens=None,
                     max_context: int = 0):
    """Absorbed latent attention (all heads share one cached latent per
    token) with a sliding window and a per-head softmax sink.
    q_abs [T, H, kv_rank], q_rot [T, H, rot_dim] (strided views ok),
    cache [blocks, block, kv_rank + rot_dim].  Rows [0, num_prefill_rows)
    are prompt portions (prefill_seq_lens = python row counts per
    sequence), the rest are single decoded tokens; max_context is a host
    hint (longest sequence in the batch) for splitting keys over
    workgroups."""
    if q_abs.is_cuda:
        _require_hybrid()
        T, H, R = q_abs.shape
        out = torch.empty((T, H, R), dtype=q_abs.dtype, device=q_abs.device)
        if q_abs.dtype == torch.bfloat16 and LATENT_ATTENTION_MFMA:
            tiles = _attention_tiles(
                _hybrid.latent_attention_tile_rows(H), num_prefill_rows,
                tuple(prefill_seq_lens or ()) if num_prefill_rows else (),
                T, q_abs.device)
            ctx = max_context or 4096
            max_keys = min(window, ctx) if window > 0 else ctx
            if _hybrid.latent_attention_mfma(
                    out, q_abs, q_rot, cache, block_table, row_seq,
                    positions, tiles[0], tiles[1], sink, scale, window,
                    max_keys):
                return out
        _hybrid.latent_attention(out, q_abs, q_rot, cache, block_table,
                                 row_seq, positions, sink, scale, window)
        return out
    return torch_ref.latent_attention_ref(
        q_abs, q_rot, cache, block_table, row_seq, positions, sink, scale,
        window)


def xielu(z, pq):
    if z.is_cuda:
        _require_hybrid()
        out = torch.empty_like(z)
        _hybrid.xielu(out, z, pq)
        return out
    return torch_ref.xielu_ref(z, pq)


def relu2(z):
    if z.is_cuda:
        out = torch.empty_like(z)
        _shared_ext("relu2")(out, z)
        return out
    return torch_ref.relu2_ref(z)


def gate_heads(v, gate):
    """v [H, T, vd] (strided ok), gate [T, H] fp32 -> [T, H*vd]."""
    if v.is_cuda:
        _require_hybrid()
        H, T, vd = v.shape
        out = torch.empty((T, H * vd), dtype=v.dtype, device=v.device)
        _hybrid.gate_heads(out, v, gate)
        return out
    return torch_ref.gate_heads_ref(v, gate)


def moe_topk_route(logits, top_k: int, capacity: int = 0,
                   scale: float = 1.0):
    """logits [T, E] fp32 -> (softmax-over-chosen weights [T, K] fp32
    times `scale`,
    expert ids [T, K] int32, padded rows [T*K] int64 or None).  With
    capacity > 0 (>= T) the padded-dispatch row of every assignment,
    expert * capacity + rank, comes from the same launch.  Any K <= E <=
    64 on the GPU kernel, wider routers take the library top-k."""
    if logits.is_cuda and logits.shape[1] <= 64:
        _require_hybrid()
        T, E = logits.shape
        w = torch.empty((T, top_k), dtype=torch.float32,
                        device=logits.device)
        idx = torch.empty((T, top_k), dtype=torch.int32,
                          device=logits.device)
        dst = counts = None
        if capacity > 0:
            dst = torch.empty(T * top_k, dtype=torch.int64,
                              device=logits.device)
            counts = torch.zeros(E, dtype=torch.int32, device=logits.device)
        _hybrid.moe_topk_route(w, idx, logits, dst, counts, capacity,
                               scale)
        return w, idx, dst
    w, idx = torch_ref.moe_topk_route_ref(logits, top_k)
    return (w * scale if scale != 1.0 else w), idx, None


# ---------------------------------------------------------------------------
# Parallel-block / sigmoid-attention mechanisms (same extension, same
# typing rules: bf16 or fp32 activations, fp32 arithmetic).
# ---------------------------------------------------------------------------
GATED_ACT_SILU = torch_ref.GATED_ACT_SILU
GATED_ACT_CLAMPED = torch_ref.GATED_ACT_CLAMPED


def add_rmsnorm_pair(residual, delta_a, delta_b, w1, w2, eps: float,
                     out_dtype):
    """residual [T, D] fp32 += delta_a + delta_b (in place; either may
    be None).  Returns (rmsnorm(residual) * w1, rmsnorm(residual) * w2)
    from ONE pass and one statistic; w2 None gives (out, None)."""
    if residual.is_cuda:
        out1 = torch.empty(residual.shape, dtype=out_dtype,
                           device=residual.device)
        out2 = None if w2 is None else torch.empty_like(out1)
        _shared_ext("add_rmsnorm_pair")(out1, out2, residual, delta_a,
                                        delta_b, w1, w2, eps)
        return out1, out2
    return torch_ref.add_rmsnorm_pair_ref(residual, delta_a, delta_b, w1,
                                          w2, eps, out_dtype)


def qk_norm_append(proj, slot_mapping, kcache, vcache, qnorm_w, knorm_w,
                   v_first, lam: float, eps: float, heads: int,
                   kv_heads: int, dim: int, vdim: int):
    """Post-processing of a fused projection [T, H*dim | G*dim | G*vdim |
    ...]: RMS norm over the whole query block and over the whole key
    block, optional value blend (1-lam) v + lam v_first (v_first [T,
    G*vdim], strided rows ok), keys and values appended to the paged
    caches (keys [blocks, G, block, dim], values page-transposed
    [blocks, G, vdim, block]).  Returns the normed queries."""
    if proj.is_cuda:
        _require_hybrid()
        q = torch.empty((proj.shape[0], heads * dim), dtype=proj.dtype,
                        device=proj.device)
        _hybrid.qk_norm_append(q, proj, slot_mapping, kcache, vcache,
                               qnorm_w, knorm_w, v_first, lam, eps, heads,
                               kv_heads, dim, vdim)
        return q
    return torch_ref.qk_norm_append_ref(
        proj, slot_mapping, kcache, vcache, qnorm_w, knorm_w, v_first, lam,
        eps, heads, kv_heads, dim, vdim)


# bf16 batches run the MFMA tile kernel; off = the block-per-row kernel
# (any dtype, any sizes) for everything
SIGMOID_ATTENTION_MFMA = True


def sigmoid_attention(q, kcache, vcache, block_table, row_seq, positions,
                      dist_bias, talk, gate, scale: float, window: int,
                      num_prefill_rows: int = 0, prefill_seq_lens=None,
                      max_context: int = 0):
    """Windowed sigmoid attention over the paged cache with a bias per
    (distance, head) (dist_bias [ND, H] fp32, distances from ND-1 on
    share the last row), the heads' weights mixed by talk [H, H], grouped
    key/value heads, and a sigmoid output gate (gate [T, H*vdim]
    pre-activations, strided rows ok).  q [T, H*dim]; returns [T,
    H*vdim].  Rows [0, num_prefill_rows) are prompt portions
    (prefill_seq_lens = python row counts per sequence), the rest single
    decoded tokens; every row reads its keys from the cache.
    max_context is a host hint (longest sequence in the batch) for
    splitting keys over workgroups."""
    if q.is_cuda:
        _require_hybrid()
        T = q.shape[0]
        H = talk.shape[0]
        out = torch.empty((T, H * vcache.shape[2]), dtype=q.dtype,
                          device=q.device)
        if q.dtype == torch.bfloat16 and SIGMOID_ATTENTION_MFMA:
            tq = _hybrid.sigmoid_attention_tile_rows()
            tiles = _attention_tiles(
                tq, num_prefill_rows,
                tuple(prefill_seq_lens or ()) if num_prefill_rows else (),
                T, q.device)
            ctx = max_context or 4096
            max_keys = min(window, ctx) if window > 0 else ctx
            if _hybrid.sigmoid_attention_mfma(
                    out, q, kcache, vcache, block_table, row_seq, positions,
                    tiles[0], tiles[1], dist_bias, talk, gate, scale,
                    window, max_keys, num_prefill_rows):
                return out
        _hybrid.sigmoid_attention(out, q, kcache, vcache, block_table,
                                  row_seq, positions, dist_bias, talk, gate,
                                  scale, window)
        return out
    return torch_ref.sigmoid_attention_ref(
        q, kcache, vcache, block_table, row_seq, positions, dist_bias, talk,
        gate, scale, window)


def gated_act(gate_up, mode: int, limit: float = 0.0, alpha: float = 1.0):
    """(gate | up) halves of the last dim -> one activation:
    GATED_ACT_SILU silu(g) * u; GATED_ACT_CLAMPED with g' = min(g, limit),
    u' = clamp(u, -limit, limit): g' * sigmoid(alpha g') * (u' + 1)."""
    if gate_up.is_cuda:
        f = gate_up.shape[-1] // 2
        out = torch.empty((*gate_up.shape[:-1], f), dtype=gate_up.dtype,
                          device=gate_up.device)
        _shared_ext("gated_act")(out, gate_up, mode, limit, alpha)
        return out
    return torch_ref.gated_act_ref(gate_up, mode, limit, alpha)


# ---------------------------------------------------------------------------
# Recurrent mixers (extension _recurrent, CPU versions in recurrent_ref):
# matrix memories, state-space layers, decayed outer-product memories,
# short convolutions, and softmax attention with a score cap.  Every op
# takes the ragged-batch description of ForwardBatch (seq_cu, seq_start,
# seq_slots) and keeps per-sequence state in slot buffers; a sequence
# whose first row is position 0 starts from zero.
# ---------------------------------------------------------------------------
from . import recurrent_ref  # noqa: E402

DECAY_LINEAR = recurrent_ref.DECAY_LINEAR
DECAY_EXP_NEG_EXP = recurrent_ref.DECAY_EXP_NEG_EXP
GATE_SIGMOID = recurrent_ref.GATE_SIGMOID
GATE_SILU = recurrent_ref.GATE_SILU


def embed_pair_norm(token_ids, positions, prev_tok, seq_cu, seq_start,
                    seq_slots, row_seq, embed, pair, pos, norm_w,
                    scale: float, buckets: int, mul_prev: int, mul_cur: int,
                    eps: float):
    """fp32 residual [T, D] = rmsnorm(embed[tok] * scale + pair[hash(prev,
    tok)] + pos[position]) * norm_w.  hash = (prev * mul_prev + tok *
    mul_cur) mod buckets; a sequence's first token reads row `buckets`.
    prev_tok [slots, 1] int32 carries each sequence's last token."""
    if embed.is_cuda:
        _require_recurrent()
        out = torch.empty((token_ids.shape[0], embed.shape[1]),
                          dtype=torch.float32, device=embed.device)
        _recurrent.embed_pair_norm(out, token_ids, positions, prev_tok,
                                   seq_cu, seq_start, seq_slots, row_seq,
                                   embed, pair, pos, norm_w, scale, buckets,
                                   mul_prev, mul_cur, eps)
        return out
    return recurrent_ref.embed_pair_norm_ref(
        token_ids, positions, prev_tok, seq_cu, seq_start, seq_slots, embed,
        pair, pos, norm_w, scale, buckets, mul_prev, mul_cur, eps)


def causal_conv(x, w, bias, state, seq_cu, seq_start, seq_slots, row_seq,
                silu: bool):
    """Per-channel causal filter over each sequence's rows: x [T, C]
    (strided rows ok), w [C, taps] fp32 (last tap = current row), bias
    [C] fp32 or None, optional silu.  state [slots, (taps-1)*C] fp32
    holds every sequence's last taps-1 inputs."""
    if x.is_cuda:
        _require_recurrent()
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _recurrent.causal_conv(out, x, w, bias, state, seq_cu, seq_start,
                               seq_slots, row_seq, silu)
        return out
    return recurrent_ref.causal_conv_ref(x, w, bias, state, seq_cu,
                                         seq_start, seq_slots, silu)


def token_shift_mix(h, mu, state, seq_cu, seq_start, seq_slots, row_seq):
    """[S, T, D]: h + (h_prev - h) * mu[s] for each of the S mixing
    vectors; h_prev = previous row of the sequence (state [slots, D] fp32
    across steps, zeros at position 0)."""
    if h.is_cuda:
        _require_recurrent()
        out = torch.empty((mu.shape[0],) + tuple(h.shape), dtype=h.dtype,
                          device=h.device)
        _recurrent.token_shift_mix(out, h, mu, state, seq_cu, seq_start,
                                   seq_slots, row_seq)
        return out
    return recurrent_ref.token_shift_mix_ref(h, mu, state, seq_cu,
                                             seq_start, seq_slots)


def mlstm_gates(pre, cap: float, m_state, seq_cu, seq_start, seq_slots):
    """Stabilised exponential gates of a matrix memory from fp32
    pre-activations [T, 2H] (input | forget); m_state [slots, H] fp32 is
    the running maximum.  Returns fp32 (decay, kscale, floor) [T, H]."""
    if pre.is_cuda:
        _require_recurrent()
        T, H = pre.shape[0], pre.shape[1] // 2
        out = torch.empty((3, T, H), dtype=torch.float32, device=pre.device)
        _recurrent.mlstm_gates(out, pre, cap, m_state, seq_cu, seq_start,
                               seq_slots)
        return out[0], out[1], out[2]
    return recurrent_ref.mlstm_gates_ref(pre, cap, m_state, seq_cu,
                                         seq_start, seq_slots)


def ssm_gates(dt_pre, a_log):
    """Step sizes and decays of a state-space layer from fp32
    pre-activations [T, H] (bias included): dt = softplus(dt_pre), decay =
    exp(-exp(a_log) * dt).  Returns fp32 (decay, dt)."""
    if dt_pre.is_cuda:
        _require_recurrent()
        out = torch.empty((2,) + tuple(dt_pre.shape), dtype=torch.float32,
                          device=dt_pre.device)
        _recurrent.ssm_gates(out, dt_pre, a_log)
        return out[0], out[1]
    dt = torch.nn.functional.softplus(dt_pre, threshold=40.0)
    return torch.exp(-torch.exp(a_log) * dt), dt


def outer_scan(q, k, v, decay, kscale, bonus, skip, state, seq_cu,
               seq_start, seq_slots, seq_rows, decay_mode: int = 0,
               ones_col: bool = False, qscale: float = 1.0):
    """Outer-product memory per (sequence, head), S [N, PP] fp32 in
    state [slots, H*N*PP]:  S' = diag(a_t) S + (kscale_t k_t) v_t^T;
    o_t = S'^T q_t, or with `bonus` u [H, N] the look-before-write form
    o_t = (S + diag(u) k_t v_t^T)^T q_t; o_t = o_t * qscale + skip_h v_t.
    q, k [T, G, N] (strided ok; head h reads group h // (H/G)), v [T, H,
    P], decay fp32 [T, H, 1 | N] holding a_t (DECAY_LINEAR) or x with a_t
    = exp(-exp(x)) (DECAY_EXP_NEG_EXP).  ones_col keeps one more memory
    column fed with ones (PP = P + 1: the normaliser n_t = a n + c k).
    Returns (o fp32 [T, H, P], n_t . q_t * qscale fp32 [T, H] or None).
    seq_rows: python row counts (host side)."""
    if v.is_cuda:
        _require_recurrent()
        T, H, P = v.shape
        out = torch.empty((T, H, P), dtype=torch.float32, device=v.device)
        norm = (torch.empty((T, H), dtype=torch.float32, device=v.device)
                if ones_col else None)
        _recurrent.outer_scan(out, norm, q, k, v, decay, kscale, bonus,
                              skip, state, seq_cu, seq_start, seq_slots,
                              decay_mode, ones_col, qscale)
        return out, norm
    return recurrent_ref.outer_scan_ref(
        q, k, v, decay, kscale, bonus, skip, state, seq_cu, seq_start,
        seq_slots, decay_mode, ones_col, qscale)


def head_norm_gate(o, gate, w, eps: float, group: int, gate_act: int,
                   gate_first: bool, den, floor, out_dtype):
    """Epilogue of a memory read-out o fp32 [T, H, P]: optional division
    of every head by max(|den|, floor) + 1e-6 (den, floor [T, H] fp32;
    floor None = 0), RMS norm in groups of `group` channels times w [C]
    fp32, and a sigmoid or silu gate from pre-activations gate [T, C]
    (strided ok) applied before or after the norm.  Returns [T, C] in
    out_dtype."""
    if o.is_cuda:
        _require_recurrent()
        T, H, P = o.shape
        out = torch.empty((T, H * P), dtype=out_dtype, device=o.device)
        _recurrent.head_norm_gate(out, o, gate, w, eps, group, gate_act,
                                  gate_first, den, floor)
        return out
    return recurrent_ref.head_norm_gate_ref(o, gate, w, eps, group, gate_act,
                                            gate_first, den, floor,
                                            out_dtype)


def append_paged_kv(k, v, kcache, vcache, slot_mapping):
    """k [T, G*N], v [T, G*P] (strided rows ok) into paged caches
    [blocks, G, block, N] and [blocks, G, block, P]."""
    if k.is_cuda:
        _require_recurrent()
        _recurrent.append_paged_kv(k, v, kcache, vcache, slot_mapping)
        return
    recurrent_ref.append_paged_kv_ref(k, v, kcache, vcache, slot_mapping)


# bf16 batches run the MFMA tile kernel when the sizes fit; off = the
# wave-per-(row, head) kernel for everything
SOFTCAP_ATTENTION_MFMA = True


@functools.lru_cache(maxsize=256)
def _softcap_tiles(seq_lens: tuple, num_seqs: int, device):
    """Tile map of the MFMA attention kernel: prompt portions (the first
    len(seq_lens) sequences of the batch) cut into runs of its tile rows,
    and the sequences that bring one decoded row.  Cached: serving
    repeats the same batch shapes."""
    tq = int(_recurrent.softcap_attention_tile_rows())
    tseq, toff = torch_ref.make_prefill_tiles(seq_lens, tq, device)
    dec = torch.arange(len(seq_lens), num_seqs, dtype=torch.int32,
                       device=device)
    return tseq, toff, dec


def softcap_attention(q, kcache, vcache, block_table, row_seq, positions,
                      scale: float, softcap: float = 0.0,
                      temp_coef: float = 0.0, temp_every: int = 1,
                      window: int = 0, num_prefill_rows: int = 0,
                      prefill_seq_lens=None, seq_cu=None, seq_start=None,
                      slopes=None, chunk: int = 0, sinks=None, gate=None):
    """Causal softmax attention over paged keys/values with grouped
    heads and separate key and value widths.  score = (q . k) * scale *
    (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)), squashed by
    softcap * tanh(. / softcap) when softcap > 0; window > 0 keeps the
    last `window` keys.  Optional: slopes [H] fp32 take slope_h * (p - j)
    off the score of key j; chunk > 0 keeps only the keys from floor(p /
    chunk) * chunk on; sinks [H] fp32 add exp(sink_h) to the softmax
    denominator (a key with that score and no value); gate [T, H*P]
    (strided rows ok) multiplies the result by sigmoid(gate).
    q [T, H*N] (strided ok) -> [T, H*P].  Rows [0,
    num_prefill_rows) are prompt portions (prefill_seq_lens = python row
    counts of the first sequences), the rest single decoded tokens;
    seq_cu / seq_start describe the sequences (needed by the tile
    kernel; without them every batch runs the row kernel)."""
    if q.is_cuda:
        _require_recurrent()
        T = q.shape[0]
        H = q.shape[1] // kcache.shape[3]
        out = torch.empty((T, H * vcache.shape[3]), dtype=q.dtype,
                          device=q.device)
        if (q.dtype == torch.bfloat16 and SOFTCAP_ATTENTION_MFMA
                and seq_cu is not None and seq_start is not None):
            lens = tuple(prefill_seq_lens or ()) if num_prefill_rows else ()
            tseq, toff, dec = _softcap_tiles(lens, seq_start.shape[0],
                                             q.device)
            if _recurrent.softcap_attention_mfma(
                    out, q, kcache, vcache, block_table, seq_cu, seq_start,
                    tseq, toff, dec, scale, softcap, temp_coef, temp_every,
                    window, slopes, chunk, sinks, gate):
                return out
        _recurrent.softcap_attention(out, q, kcache, vcache, block_table,
                                     row_seq, positions, scale, softcap,
                                     temp_coef, temp_every, window, slopes,
                                     chunk, sinks, gate)
        return out
    return recurrent_ref.softcap_attention_ref(
        q, kcache, vcache, block_table, row_seq, positions, scale, softcap,
        temp_coef, temp_every, window, slopes, chunk, sinks, gate)


def qk_norm_rope_append(proj, positions, slot_mapping, kcache, vcache,
                        qnorm_w, knorm_w, inv_freq, mag: float, eps: float,
                        heads: int, kv_heads: int, dim: int, vdim: int):
    """Post-processing of a fused projection [T, heads*dim | kv_heads*dim
    | kv_heads*vdim | ...] (strided rows ok): per-head RMS norm of the
    queries and keys (weights [dim] fp32 shared by the heads; None = no
    norm), interleaved-pair rotation of each head's first
    2*len(inv_freq) entries by position * inv_freq (fp32 angles, cos and
    sin times `mag`; inv_freq None = no rotation), keys and values
    appended to the paged caches [blocks, kv_heads, block, dim | vdim].
    Returns the queries [T, heads*dim]."""
    if proj.is_cuda:
        _require_recurrent()
        q = torch.empty((proj.shape[0], heads * dim), dtype=proj.dtype,
                        device=proj.device)
        _recurrent.qk_norm_rope_append(q, proj, positions, slot_mapping,
                                       kcache, vcache, qnorm_w, knorm_w,
                                       inv_freq, mag, eps, heads, kv_heads,
                                       dim, vdim)
        return q
    return recurrent_ref.qk_norm_rope_append_ref(
        proj, positions, slot_mapping, kcache, vcache, qnorm_w, knorm_w,
        inv_freq, mag, eps, heads, kv_heads, dim, vdim)


def decay_beta_gates(pre, a_log, dt_bias):
    """Gates of a delta-rule memory from fp32 pre-activations [T, 2H]
    (step | write strength): decay = exp(-exp(a_log) * softplus(step +
    dt_bias)), beta = sigmoid(write strength).  Returns fp32 (decay,
    beta), each [T, H]."""
    if pre.is_cuda:
        _require_recurrent()
        T, H = pre.shape[0], pre.shape[1] // 2
        out = torch.empty((2, T, H), dtype=torch.float32, device=pre.device)
        _recurrent.decay_beta_gates(out, pre, a_log, dt_bias)
        return out[0], out[1]
    return recurrent_ref.decay_beta_gates_ref(pre, a_log, dt_bias)


def delta_scan(q, k, v, decay, beta, state, seq_cu, seq_start, seq_slots,
               seq_rows, unit_eps: float = 0.0, qscale: float = 1.0):
    """Gated delta-rule memory per (sequence, head), S [N, P] fp32 in
    state [slots, H*N*P].  Per row, in this order: S <- a_t S; u = b_t
    (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t.  With unit_eps > 0
    q and k are first scaled to unit length per head (x / sqrt(sum x^2 +
    unit_eps)); q is multiplied by qscale.  q, k [T, G, N] (strided ok;
    head h reads group h // (H/G)), v [T, H, P], decay and beta fp32 [T,
    H].  Returns o fp32 [T, H, P].  seq_rows: python row counts."""
    if v.is_cuda:
        _require_recurrent()
        T, H, P = v.shape
        out = torch.empty((T, H, P), dtype=torch.float32, device=v.device)
        _recurrent.delta_scan(out, q, k, v, decay, beta, state, seq_cu,
                              seq_start, seq_slots, unit_eps, qscale)
        return out
    return recurrent_ref.delta_scan_ref(q, k, v, decay, beta, state, seq_cu,
                                        seq_start, seq_slots, unit_eps,
                                        qscale)


def moe_group_route(logits, correction, top_k: int, groups: int, keep: int,
                    capacity: int = 0):
    """Sigmoid router with a selection-only correction and expert
    groups: logits [T, E] fp32, correction [E] fp32 -> (weights [T, K]
    fp32 = sigmoid(logit) of the chosen experts, not renormalised; expert
    ids [T, K] int32; padded rows [T*K] int64 or None).  Choice score =
    sigmoid(logit) + correction; the E experts form `groups` equal runs
    of neighbours, a group scores the sum of its two best choice scores
    and only the `keep` best groups can be chosen from.  With capacity >
    0 (>= T) the padded-dispatch row of every assignment, expert *
    capacity + rank, comes from the same launch.  E <= 64 on the GPU
    kernel."""
    if logits.is_cuda and logits.shape[1] <= 64:
        _require_recurrent()
        T, E = logits.shape
        w = torch.empty((T, top_k), dtype=torch.float32,
                        device=logits.device)
        idx = torch.empty((T, top_k), dtype=torch.int32,
                          device=logits.device)
        dst = counts = None
        if capacity > 0:
            dst = torch.empty(T * top_k, dtype=torch.int64,
                              device=logits.device)
            counts = torch.zeros(E, dtype=torch.int32, device=logits.device)
        _recurrent.moe_group_route(w, idx, logits, correction, dst, counts,
                                   capacity, groups, keep)
        return w, idx, dst
    w, idx = recurrent_ref.moe_group_route_ref(logits, correction, top_k,
                                               groups, keep)
    return w, idx, None


def add_normed_rmsnorm(residual, delta, w_post, w_pre, eps: float,
                       out_dtype):
    """Sandwich-norm step: residual [T, D] fp32 += rmsnorm(delta) *
    w_post (in place; delta None = nothing added), then returns
    rmsnorm(residual) * w_pre in out_dtype (w_pre None: the residual
    itself in out_dtype).  Weights fp32 [D]."""
    if residual.is_cuda:
        _require_recurrent()
        out = torch.empty(residual.shape, dtype=out_dtype,
                          device=residual.device)
        _recurrent.add_normed_rmsnorm(out, residual, delta, w_post, w_pre,
                                      eps)
        return out
    return recurrent_ref.add_normed_rmsnorm_ref(residual, delta, w_post,
                                                w_pre, eps, out_dtype)


def gelu_mul_rows(z, table, tokens, col0: int):
    """gelu_tanh(z [T, W]) * table[tokens, col0 : col0 + W] (table rows
    gathered by token id)."""
    if z.is_cuda:
        _require_recurrent()
        out = torch.empty_like(z)
        _recurrent.gelu_mul_rows(out, z, table, tokens, col0)
        return out
    return recurrent_ref.gelu_mul_rows_ref(z, table, tokens, col0)


def rmsnorm_pair_mean(a, b, wa, wb, eps: float):
    """0.5 * (rmsnorm(a) * wa + rmsnorm(b) * wb): the two branches of a
    parallel mixer, each normed over the model width, averaged."""
    if a.is_cuda:
        _require_recurrent()
        out = torch.empty_like(a)
        _recurrent.rmsnorm_pair_mean(out, a, b, wa, wb, eps)
        return out
    return recurrent_ref.rmsnorm_pair_mean_ref(a, b, wa, wb, eps)
