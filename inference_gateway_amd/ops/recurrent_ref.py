"""CPU (torch, fp32) implementations of the recurrent-mixer ops: what the
gfx950 kernels of csrc_recurrent compute, written for clarity.  They take
the same ragged-batch description as the kernels: rows of sequence s are
[seq_cu[s], seq_cu[s+1]), its first row sits at position seq_start[s],
and its per-sequence state lives in row seq_slots[s] of a slot buffer.  A
sequence whose first row is position 0 starts from zero state whatever
its slot held.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

DECAY_LINEAR = 0        # decay tensor holds the factor itself
DECAY_EXP_NEG_EXP = 1   # decay tensor holds x; factor = exp(-exp(x))

GATE_SIGMOID = 0
GATE_SILU = 1


def _seqs(seq_cu, seq_start, seq_slots):
    cu = seq_cu.tolist()
    return [(cu[s], cu[s + 1], st, sl) for s, (st, sl) in enumerate(
        zip(seq_start.tolist(), seq_slots.tolist()))]


def embed_pair_norm_ref(token_ids, positions, prev_tok, seq_cu, seq_start,
                        seq_slots, embed, pair, pos, norm_w, scale, buckets,
                        mul_prev, mul_cur, eps):
    T = token_ids.shape[0]
    tok = token_ids.to(torch.int64)
    prev = torch.empty_like(tok)
    first = torch.zeros(T, dtype=torch.bool, device=tok.device)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        if r1 == r0:
            continue
        prev[r0 + 1:r1] = tok[r0:r1 - 1]
        if st == 0:
            prev[r0] = 0
            first[r0] = True
        else:
            prev[r0] = int(prev_tok[sl, 0])
        prev_tok[sl, 0] = int(tok[r1 - 1])
    row = (prev * mul_prev + tok * mul_cur) % buckets
    row = torch.where(first, torch.full_like(row, buckets), row)
    x = (embed[tok].float() * scale + pair[row].float()
         + pos[positions.to(torch.int64)].float())
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * norm_w


def causal_conv_ref(x, w, bias, state, seq_cu, seq_start, seq_slots, silu):
    """x [T, C] (any row stride), w [C, taps] fp32 with the LAST tap on
    the current row, state [slots, (taps-1)*C] fp32 = the sequence's
    last taps-1 inputs, oldest first."""
    T, C = x.shape
    taps = w.shape[1]
    xf = x.float()
    out = torch.empty((T, C), dtype=torch.float32, device=x.device)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        if r1 == r0:
            continue
        hist = (state[sl, :(taps - 1) * C].view(taps - 1, C).clone()
                if st > 0 else
                torch.zeros((taps - 1, C), dtype=torch.float32,
                            device=x.device))
        u = torch.cat([hist, xf[r0:r1]], 0)          # [taps-1 + n, C]
        acc = torch.zeros((r1 - r0, C), dtype=torch.float32,
                          device=x.device)
        for j in range(taps):
            acc += w[:, j] * u[j:j + r1 - r0]
        out[r0:r1] = acc
        if taps > 1:
            state[sl] = u[-(taps - 1):].reshape(-1)
    if bias is not None:
        out += bias
    if silu:
        out = F.silu(out)
    return out.to(x.dtype)


def token_shift_mix_ref(h, mu, state, seq_cu, seq_start, seq_slots):
    """out[s] = h + (h_prev - h) * mu[s]; h_prev is the previous row of
    the same sequence (slot state across steps, zeros at position 0)."""
    hf = h.float()
    prev = torch.empty_like(hf)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        if r1 == r0:
            continue
        prev[r0 + 1:r1] = hf[r0:r1 - 1]
        prev[r0] = state[sl] if st > 0 else 0.0
        state[sl] = hf[r1 - 1]
    return (hf[None] + (prev - hf)[None] * mu[:, None, :]).to(h.dtype)


def mlstm_gates_ref(pre, cap, m_state, seq_cu, seq_start, seq_slots):
    """pre [T, 2H] fp32 = (input | forget) gate pre-activations.  With
    i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)) and the
    running maximum m (0 at the sequence start): returns decay =
    exp(f + m_prev - m), kscale = exp(i - m), floor = exp(-m)."""
    T, H2 = pre.shape
    H = H2 // 2
    gi = cap * torch.tanh(pre[:, :H] / cap)
    gf = F.logsigmoid(cap * torch.tanh(pre[:, H:] / cap))
    decay = torch.empty((T, H), dtype=torch.float32, device=pre.device)
    kscale = torch.empty_like(decay)
    floor = torch.empty_like(decay)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        m = m_state[sl].clone() if st > 0 else torch.zeros(
            H, dtype=torch.float32, device=pre.device)
        for t in range(r0, r1):
            m_new = torch.maximum(gf[t] + m, gi[t])
            decay[t] = torch.exp(gf[t] + m - m_new)
            kscale[t] = torch.exp(gi[t] - m_new)
            floor[t] = torch.exp(-m_new)
            m = m_new
        if r1 > r0:
            m_state[sl] = m
    return decay, kscale, floor


def outer_scan_ref(q, k, v, decay, kscale, bonus, skip, state, seq_cu,
                   seq_start, seq_slots, decay_mode, ones_col, qscale):
    """Matrix memory per (sequence, head): S [N, PP] fp32, PP = P (+1
    column fed with ones when ones_col).
      S' = diag(a_t) S + (kscale_t k_t) v_t^T
      bonus None:  o_t = S'^T q_t              (reads the updated memory)
      bonus u:     o_t = (S + diag(u) k_t v_t^T)^T q_t   (reads the old)
      o_t = o_t * qscale + skip_h * v_t
    q, k [T, G, N] (head h uses group h // (H/G)), v [T, H, P], decay
    [T, H, Nd] with Nd in {1, N}; returns fp32 (o [T, H, P], read-out of
    the ones column [T, H] or None)."""
    T, H, P = v.shape
    G, N = q.shape[1], q.shape[2]
    PP = P + (1 if ones_col else 0)
    rep = H // G
    qf = q.float().repeat_interleave(rep, 1)
    kf = k.float().repeat_interleave(rep, 1)
    vf = v.float()
    if ones_col:
        vf = torch.cat([vf, torch.ones((T, H, 1), dtype=torch.float32,
                                       device=v.device)], 2)
    a = decay.float()
    if decay_mode == DECAY_EXP_NEG_EXP:
        a = torch.exp(-torch.exp(a))
    a = a.expand(T, H, N)
    if kscale is not None:
        kf = kf * kscale[:, :, None]
    out = torch.empty((T, H, PP), dtype=torch.float32, device=v.device)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        if r1 == r0:
            continue
        S = (state[sl].view(H, N, PP).clone() if st > 0 else torch.zeros(
            (H, N, PP), dtype=torch.float32, device=v.device))
        for t in range(r0, r1):
            kv = kf[t][:, :, None] * vf[t][:, None, :]
            if bonus is None:
                S = a[t][:, :, None] * S + kv
                out[t] = torch.einsum("hnp,hn->hp", S, qf[t])
            else:
                out[t] = torch.einsum(
                    "hnp,hn->hp", S + bonus[:, :, None] * kv, qf[t])
                S = a[t][:, :, None] * S + kv
        state[sl] = S.reshape(-1)
    out = out * qscale
    if skip is not None:
        out[:, :, :P] += skip[None, :, None] * v.float()
    if ones_col:
        return out[:, :, :P].contiguous(), out[:, :, P].contiguous()
    return out, None


def head_norm_gate_ref(o, gate, w, eps, group, gate_act, gate_first, den,
                       floor, out_dtype):
    """o fp32 [T, H, P].  With den [T, H]: o <- o / (max(|den|, floor) +
    1e-6) per head (floor None = 0).  Then, over the flattened channels
    C = H*P: gate (sigmoid or silu of the pre-activations `gate` [T, C])
    before or after an RMS norm in groups of `group` channels, times w."""
    T, H, P = o.shape
    if den is not None:
        d = den.abs()
        if floor is not None:
            d = torch.maximum(d, floor)
        o = o / (d + 1e-6)[:, :, None]
    y = o.reshape(T, -1)
    C = y.shape[1]
    g = gate.float()
    g = torch.sigmoid(g) if gate_act == GATE_SIGMOID else F.silu(g)
    if gate_first:
        y = y * g
    yg = y.view(T, C // group, group)
    y = (yg * torch.rsqrt((yg * yg).mean(-1, keepdim=True) + eps)
         ).reshape(T, C) * w
    if not gate_first:
        y = y * g
    return y.to(out_dtype)


def append_paged_kv_ref(k, v, kcache, vcache, slot_mapping):
    """k [T, G*N], v [T, G*P] -> caches [blocks, G, block, N|P]."""
    nb, G, bs, N = kcache.shape
    P = vcache.shape[3]
    sm = slot_mapping.to(torch.int64)
    blk, off = sm // bs, sm % bs
    kcache[blk, :, off] = k.reshape(-1, G, N).to(kcache.dtype)
    vcache[blk, :, off] = v.reshape(-1, G, P).to(vcache.dtype)


def softcap_attention_ref(q, kcache, vcache, block_table, row_seq,
                          positions, scale, softcap, temp_coef, temp_every,
                          window, slopes=None, chunk=0, sinks=None,
                          gate=None):
    """Causal softmax attention of every row against its sequence's
    paged keys 0..position (the last `window` of them when window > 0).
    score = (q . k) * scale * temp(p), temp(p) = 1 + temp_coef *
    ln(floor((p + 1) / temp_every) + 1); then softcap * tanh(score /
    softcap) when softcap > 0.  slopes [H]: slope_h * (p - j) is taken
    off the score of key j.  chunk > 0: only keys from floor(p / chunk) *
    chunk on.  sinks [H]: exp(sink_h) joins the softmax denominator (a
    key with that score and no value).  gate [T, H*P]: the result is
    multiplied by sigmoid(gate).  q [T, H*N] -> [T, H*P]."""
    nb, G, bs, N = kcache.shape
    P = vcache.shape[3]
    T = q.shape[0]
    H = q.shape[1] // N
    rep = H // G
    qf = q.float().view(T, H, N)
    out = torch.empty((T, H, P), dtype=torch.float32, device=q.device)
    pos_l = positions.tolist()
    seq_l = row_seq.tolist()
    for t in range(T):
        p = pos_l[t]
        lo = max(0, p - window + 1) if window > 0 else 0
        if chunk > 0:
            lo = max(lo, p // chunk * chunk)
        j = torch.arange(lo, p + 1, device=q.device)
        blocks = block_table[seq_l[t]].to(torch.int64)[j // bs]
        kk = kcache[blocks, :, j % bs].float()      # [n, G, N]
        vv = vcache[blocks, :, j % bs].float()      # [n, G, P]
        kk = kk.repeat_interleave(rep, 1)
        vv = vv.repeat_interleave(rep, 1)
        temp = 1.0 + temp_coef * math.log((p + 1) // temp_every + 1.0)
        s = torch.einsum("hn,jhn->hj", qf[t], kk) * (scale * temp)
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if slopes is not None:
            s = s - slopes[:, None] * (p - j).float()[None, :]
        if sinks is not None:
            w = torch.softmax(torch.cat([s, sinks[:, None]], 1), -1)[:, :-1]
        else:
            w = torch.softmax(s, -1)
        out[t] = torch.einsum("hj,jhp->hp", w, vv)
    out = out.reshape(T, H * P)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(q.dtype)


def qk_norm_rope_append_ref(proj, positions, slot_mapping, kcache, vcache,
                            qnorm_w, knorm_w, inv_freq, mag, eps, heads,
                            kv_heads, dim, vdim):
    """proj [T, heads*dim | kv_heads*dim | kv_heads*vdim | ...]: every
    query and key head is RMS-normed over its dim entries (weights [dim]
    shared by the heads; None = no norm), then pairs (2i, 2i+1) of its
    first 2*len(inv_freq) entries turn by position * inv_freq[i] with cos
    and sin times `mag` (inv_freq None = no rotation).  Keys and values
    go to the paged caches; the queries are returned [T, heads*dim]."""
    T = proj.shape[0]
    nq, nk = heads * dim, kv_heads * dim
    q = proj[:, :nq].float().reshape(T, heads, dim)
    k = proj[:, nq:nq + nk].float().reshape(T, kv_heads, dim)
    v = proj[:, nq + nk:nq + nk + kv_heads * vdim]

    def prep(x, w):
        if w is not None:
            x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w
        if inv_freq is not None:
            R = inv_freq.shape[0]
            ang = positions.float()[:, None] * inv_freq.float()[None, :]
            c = (torch.cos(ang) * mag)[:, None, :]
            s = (torch.sin(ang) * mag)[:, None, :]
            a, b = x[..., 0:2 * R:2], x[..., 1:2 * R:2]
            rot = torch.stack([a * c - b * s, b * c + a * s], -1)
            x = torch.cat([rot.reshape(T, x.shape[1], 2 * R),
                           x[..., 2 * R:]], -1)
        return x

    q, k = prep(q, qnorm_w), prep(k, knorm_w)
    append_paged_kv_ref(k.reshape(T, nk).to(proj.dtype), v, kcache, vcache,
                        slot_mapping)
    return q.reshape(T, nq).to(proj.dtype)


def decay_beta_gates_ref(pre, a_log, dt_bias):
    """pre [T, 2H] fp32 = (step | write-strength) pre-activations:
    decay = exp(-exp(a_log) * softplus(step + dt_bias)), beta =
    sigmoid(write-strength).  Returns fp32 ([T, H], [T, H])."""
    H = pre.shape[1] // 2
    dt = F.softplus(pre[:, :H] + dt_bias, threshold=40.0)
    return torch.exp(-torch.exp(a_log) * dt), torch.sigmoid(pre[:, H:])


def delta_scan_ref(q, k, v, decay, beta, state, seq_cu, seq_start,
                   seq_slots, unit_eps, qscale):
    """Gated delta-rule memory per (sequence, head), S [N, P] fp32 in
    state [slots, H*N*P].  With unit_eps > 0, q and k are first scaled
    to unit length per head, x / sqrt(sum x^2 + unit_eps); q is then
    multiplied by qscale.  Per row, in this order:
      S <- a_t S;  u = b_t (v_t - S^T k_t);  S <- S + k_t u^T;
      o_t = S^T q_t.
    q, k [T, G, N] (head h uses group h // (H/G)), v [T, H, P], decay and
    beta fp32 [T, H]; returns o fp32 [T, H, P]."""
    T, H, P = v.shape
    G, N = q.shape[1], q.shape[2]
    rep = H // G
    qf, kf = q.float(), k.float()
    if unit_eps > 0:
        qf = qf * torch.rsqrt((qf * qf).sum(-1, keepdim=True) + unit_eps)
        kf = kf * torch.rsqrt((kf * kf).sum(-1, keepdim=True) + unit_eps)
    qf = (qf * qscale).repeat_interleave(rep, 1)
    kf = kf.repeat_interleave(rep, 1)
    vf = v.float()
    out = torch.empty((T, H, P), dtype=torch.float32, device=v.device)
    for r0, r1, st, sl in _seqs(seq_cu, seq_start, seq_slots):
        if r1 == r0:
            continue
        S = (state[sl].view(H, N, P).clone() if st > 0 else torch.zeros(
            (H, N, P), dtype=torch.float32, device=v.device))
        for t in range(r0, r1):
            S = S * decay[t][:, None, None]
            u = beta[t][:, None] * (vf[t] - torch.einsum(
                "hnp,hn->hp", S, kf[t]))
            S = S + kf[t][:, :, None] * u[:, None, :]
            out[t] = torch.einsum("hnp,hn->hp", S, qf[t])
        state[sl] = S.reshape(-1)
    return out


def moe_group_route_ref(logits, correction, top, groups, keep):
    """logits [T, E] fp32 -> (weights [T, top] fp32, ids [T, top] int32).
    Scores s = sigmoid(logits); choice scores c = s + correction.  The E
    experts are `groups` equal runs of neighbours; a group's score is the
    sum of its two largest choice scores (its only one when it has a
    single expert) and only experts of the `keep` best groups can be
    chosen; the `top` largest choice scores among them are taken and
    weighted by their s (not renormalised)."""
    T, E = logits.shape
    s = torch.sigmoid(logits.float())
    c = s + correction.float()
    if groups > 1:
        size = E // groups
        cg = c.view(T, groups, size)
        gscore = cg.topk(min(2, size), -1).values.sum(-1)
        kept = gscore.topk(keep, -1).indices
        mask = torch.zeros((T, groups), dtype=torch.bool,
                           device=logits.device)
        mask.scatter_(1, kept, True)
        c = torch.where(mask[:, :, None], cg,
                        torch.full_like(cg, float("-inf"))).reshape(T, E)
    idx = c.topk(top, -1).indices
    return s.gather(1, idx), idx.to(torch.int32)


def add_normed_rmsnorm_ref(residual, delta, w_post, w_pre, eps, out_dtype):
    """residual [T, D] fp32 += rmsnorm(delta) * w_post (in place; delta
    None = nothing added); returns rmsnorm(residual) * w_pre in
    out_dtype, or the residual itself in out_dtype when w_pre is None."""
    if delta is not None:
        d = delta.float()
        residual += d * torch.rsqrt((d * d).mean(-1, keepdim=True)
                                    + eps) * w_post
    if w_pre is None:
        return residual.to(out_dtype)
    return (residual * torch.rsqrt((residual * residual).mean(
        -1, keepdim=True) + eps) * w_pre).to(out_dtype)


def gelu_mul_rows_ref(z, table, tokens, col0):
    """gelu_tanh(z [T, W]) * table[tokens, col0 : col0 + W]."""
    W = z.shape[1]
    e = table[tokens.to(torch.int64), col0:col0 + W].float()
    return (F.gelu(z.float(), approximate="tanh") * e).to(z.dtype)


def rmsnorm_pair_mean_ref(a, b, wa, wb, eps):
    """0.5 * (a / rms(a) * wa + b / rms(b) * wb), row by row."""
    af, bf = a.float(), b.float()
    ya = af * torch.rsqrt((af * af).mean(-1, keepdim=True) + eps) * wa
    yb = bf * torch.rsqrt((bf * bf).mean(-1, keepdim=True) + eps) * wb
    return (0.5 * (ya + yb)).to(a.dtype)
