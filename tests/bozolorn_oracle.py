"""Plain float64 model of the Bozolorn design, token by token, one
function per mechanism.  It shares no code with the engine: weights come
in as a dict of numpy arrays under the checkpoint's tensor names, the
configuration as the parsed config.json dict.

Notation: D model width, T tokens of ONE sequence, H query heads, G
key/value heads, N query/key entries per head, P value entries per head.
"""
from __future__ import annotations

import math

import numpy as np


def rms_unit(x, eps):
    """x scaled to unit root mean square over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return np.logaddexp(0.0, x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi)
                                    * (z + 0.044715 * z ** 3)))


# ---------------------------------------------------------------------------
# attention with a linear distance bias inside position chunks
# ---------------------------------------------------------------------------
def distance_slopes(H):
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


def chunk_bias_attention(q, k, v, H, G, scale, chunk):
    """q [T, H, N], k [T, G, N], v [T, G, P].  Position i attends to
    j <= i of its own chunk of `chunk` positions (counted from the start
    of the sequence); score = q.k * scale - slope_h * (i - j)."""
    T = q.shape[0]
    slopes = distance_slopes(H)
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        lo = (i // chunk) * chunk if chunk else 0
        for h in range(H):
            g = h // (H // G)
            s = np.array([q[i, h] @ k[j, g] * scale - slopes[h] * (i - j)
                          for j in range(lo, i + 1)])
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ v[lo:i + 1, g]
    return out


def attention_mixer(h, W, pre, m, kv=None):
    """Returns (output, (k, v)); `kv` given = keys and values borrowed
    from another layer (this layer then has no k/v projections)."""
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).reshape(T, H, N)
    if kv is None:
        kv = ((h @ W[pre + "k"].T).reshape(T, G, N),
              (h @ W[pre + "v"].T).reshape(T, G, P))
    o = chunk_bias_attention(q, kv[0], kv[1], H, G, m["scale"],
                             (m.get("mask") or {}).get("size", 0))
    o = o.reshape(T, H * P) * sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T, kv


# ---------------------------------------------------------------------------
# rotated attention with a unit sink in the denominator
# ---------------------------------------------------------------------------
def rotary_frequencies(rot):
    """Angular step per pair i of the rotated dimensions, and the factor
    on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return np.array(f), 1.0

    def where(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) \
            / (2.0 * math.log(base))

    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * ramp + fi * (1.0 - ramp))
    return np.array(out), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_pairs(x, rot):
    """x [T, heads, N]: entries (2i, 2i+1) of the first rot.dims are
    turned by position * frequency_i; the rest pass."""
    freq, mag = rotary_frequencies(rot)
    y = x.copy()
    for p in range(x.shape[0]):
        for i, f in enumerate(freq):
            c, s = math.cos(p * f) * mag, math.sin(p * f) * mag
            a, b = x[p, :, 2 * i], x[p, :, 2 * i + 1]
            y[p, :, 2 * i] = a * c - b * s
            y[p, :, 2 * i + 1] = b * c + a * s
    return y


def sink_attention(q, k, v, H, G, scale):
    """Causal; p_j = exp(s_j) / (1 + sum exp(s_j))."""
    T = q.shape[0]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        for h in range(H):
            g = h // (H // G)
            s = k[:i + 1, g] @ q[i, h] * scale
            m = max(s.max(), 0.0)
            p = np.exp(s - m)
            out[i, h] = (p / (math.exp(-m) + p.sum())) @ v[:i + 1, g]
    return out


def left_mixer(h, W, pre, m, eps):
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).reshape(T, H, N)
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).reshape(T, G, N)
    v = (h @ W[pre + "v"].T + W[pre + "v.b"]).reshape(T, G, P)
    q = rms_unit(q, eps) * W[pre + "q.norm"]
    k = rms_unit(k, eps) * W[pre + "k.norm"]
    if m.get("rot"):
        q, k = rotate_pairs(q, m["rot"]), rotate_pairs(k, m["rot"])
    o = sink_attention(q, k, v, H, G, m["scale"])
    return o.reshape(T, H * P) @ W[pre + "o"].T


# ---------------------------------------------------------------------------
# gated delta rule
# ---------------------------------------------------------------------------
def short_conv(u, w):
    """Per-channel causal filter: the LAST tap multiplies the current
    token, zeros before the sequence starts.  u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def delta_rule(q, k, v, beta, g):
    """q, k [T, H, N], v [T, H, P], beta, g [T, H].  Per head, in this
    order: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, N = q.shape
    P = v.shape[2]
    S = np.zeros((H, N, P))
    o = np.zeros((T, H, P))
    for t in range(T):
        for hd in range(H):
            S[hd] *= g[t, hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ k[t, hd])
            S[hd] += np.outer(k[t, hd], u)
            o[t, hd] = S[hd].T @ q[t, hd]
    return o


def right_mixer(h, W, pre, m, eps):
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ W[pre + "q"].T, W[pre + "q.conv"]))
    k = silu(short_conv(h @ W[pre + "k"].T, W[pre + "k.conv"]))
    v = silu(short_conv(h @ W[pre + "v"].T, W[pre + "v.conv"]))
    q, k = q.reshape(T, G, N), k.reshape(T, G, N)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * N ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    rep = H // G
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)
    beta = sigmoid(h @ W[pre + "b"].T)
    g = np.exp(-np.exp(W[pre + "A_log"])
               * softplus(h @ W[pre + "a"].T + W[pre + "dt_bias"]))
    o = delta_rule(q, k, v.reshape(T, H, P), beta, g)
    o = rms_unit(o, eps) * W[pre + "norm"]
    o = o.reshape(T, H * P) * silu(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def parallel_mixer(h, W, pre, m, eps):
    a = left_mixer(h, W, pre + "left.", m["left"], eps)
    b = right_mixer(h, W, pre + "right.", m["right"], eps)
    return 0.5 * (rms_unit(a, eps) * W[pre + "left.out"]
                  + rms_unit(b, eps) * W[pre + "right.out"])


# ---------------------------------------------------------------------------
# routed clamped-GLU experts
# ---------------------------------------------------------------------------
def route(z, correction, top, groups, keep):
    """z [E] router logits of one token -> (expert ids, weights)."""
    s = sigmoid(z)
    choice = s + correction
    E = len(z)
    if groups and groups > 1:
        size = E // groups
        gs = [np.sort(choice[a * size:(a + 1) * size])[-2:].sum()
              for a in range(groups)]
        kept = np.argsort(gs)[::-1][:keep]
        masked = np.full(E, -np.inf)
        for a in kept:
            masked[a * size:(a + 1) * size] = choice[a * size:(a + 1) * size]
        choice = masked
    ids = np.argsort(choice)[::-1][:top]
    return ids, s[ids]


def expert(h, W, pre, limit):
    g = np.minimum(h @ W[pre + "gate"].T, limit)
    u = np.clip(h @ W[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def moe(h, W, pre, f):
    r = f["router"]
    gr = r.get("groups") or {}
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        ids, w = route(h[t] @ W[pre + "router"].T, W[pre + "correction"],
                       r["top"], gr.get("count", 1), gr.get("keep", 1))
        for e, we in zip(ids, w):
            out[t] += we * expert(h[t], W, pre + f"e{e}.",
                                  f["expert"]["limit"])
    return out


def token_side(x, tokens, W, pre, i, dim, eps):
    """What every layer adds from the token itself, after its
    feed-forward."""
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ W[pre + "gate"].T) * e) @ W[pre + "proj"].T
    return rms_unit(y, eps) * W[pre + "norm"]


def forward(W, cfg, tokens):
    """Returns (logits [T, vocab], residual after every layer
    [layers, T, D])."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    x = W["embed"][tokens] * cfg["embedding"]["scale"]
    kv_of, taps = {}, []
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        h = rms_unit(x, eps) * W[p + "norm1"]
        if l["type"] == "attention":
            src = m.get("kv_from")
            d, kv_of[i] = attention_mixer(
                h, W, p + "mix.", m, None if src is None else kv_of[src])
        elif l["type"] == "parallel":
            d = parallel_mixer(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(l["type"])
        x = x + rms_unit(d, eps) * W[p + "norm1b"]
        if l.get("mlp") is not None:
            d = moe(rms_unit(x, eps) * W[p + "norm2"], W, p + "mlp.",
                    l["mlp"])
            x = x + rms_unit(d, eps) * W[p + "norm2b"]
        if cfg.get("token_side"):
            x = x + token_side(x, tokens, W, p + "side.", i,
                               cfg["token_side"]["dim"], eps)
        taps.append(x.copy())
    logits = (rms_unit(x, eps) * W["final.norm"]) @ W["head"].T
    return logits, np.stack(taps)


# ---------------------------------------------------------------------------
# random checkpoints for the tests
# ---------------------------------------------------------------------------
def tensor_shapes(cfg):
    """Tensor name -> shape of a checkpoint of this configuration."""
    D, V = cfg["width"], cfg["vocab"]
    L = len(cfg["layers"])
    sh = {"embed": (V, D), "final.norm": (D,), "head": (V, D)}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        sh["side.embed"] = (V, side * L)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        sh.update({p + "norm1": (D,), p + "norm1b": (D,)})
        if l["type"] == "attention":
            H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            q = p + "mix."
            sh.update({q + "q": (H * N, D), q + "g": (H * P, D),
                       q + "o": (D, H * P)})
            if m.get("kv_from") is None:
                sh.update({q + "k": (G * N, D), q + "v": (G * P, D)})
        else:
            a, b = m["left"], m["right"]
            H, G, N, P = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            sh.update({q + "q": (H * N, D), q + "q.b": (H * N,),
                       q + "k": (G * N, D), q + "k.b": (G * N,),
                       q + "v": (G * P, D), q + "v.b": (G * P,),
                       q + "q.norm": (N,), q + "k.norm": (N,),
                       q + "o": (D, H * P), q + "out": (D,)})
            H, G, N, P = b["heads"], b["kv_heads"], b["dim"], b["vdim"]
            r = p + "mix.right."
            sh.update({r + "q": (G * N, D), r + "q.conv": (G * N, b["conv"]),
                       r + "k": (G * N, D), r + "k.conv": (G * N, b["conv"]),
                       r + "v": (H * P, D), r + "v.conv": (H * P, b["conv"]),
                       r + "b": (H, D), r + "a": (H, D), r + "A_log": (H,),
                       r + "dt_bias": (H,), r + "norm": (P,),
                       r + "g": (H * P, D), r + "o": (D, H * P),
                       r + "out": (D,)})
        f = l.get("mlp")
        if f is not None:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            sh.update({p + "norm2": (D,), p + "norm2b": (D,),
                       p + "mlp.router": (E, D), p + "mlp.correction": (E,)})
            for e in range(E):
                sh.update({p + f"mlp.e{e}.gate": (ff, D),
                           p + f"mlp.e{e}.up": (ff, D),
                           p + f"mlp.e{e}.down": (D, ff)})
        if side:
            sh.update({p + "side.gate": (side, D), p + "side.proj": (D, side),
                       p + "side.norm": (D,)})
    return sh


def random_weights(cfg, seed=0):
    """Random weights, rounded to bfloat16 (what a checkpoint stores),
    as float64 arrays."""
    import torch

    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        x = torch.randn(shape, generator=g, dtype=torch.float32)
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            x = x * 0.5 / cfg["embedding"]["scale"]
        elif name == "side.embed":
            x = x * 0.7
        elif last in ("norm1", "norm2", "norm1b", "norm2b", "norm", "out"):
            x = 1.0 + x * 0.2
        elif last in ("A_log", "dt_bias"):
            x = x * 0.7
        elif last == "correction":
            x = x * 0.3
        elif last == "b" and len(shape) == 1:
            x = x * 0.5
        elif last == "conv":
            x = x * 0.6
        elif len(shape) == 2:
            x = x * shape[1] ** -0.5 * (
                3.0 if last in ("router", "a", "b") else 1.5)
        W[name] = x.to(torch.bfloat16).double().numpy()
    return W


def save_checkpoint(path, cfg, W):
    """config.json + model.safetensors (bfloat16) in `path`."""
    import json
    import os

    import torch
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.from_numpy(v).to(torch.bfloat16).contiguous()
               for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return str(path)


def make_config(width, vocab, layers, side=0, scale=None, eps=1e-5):
    cfg = {"architecture": "Bozolorn", "width": width, "vocab": vocab,
           "norm": {"eps": eps},
           "embedding": {"scale": scale or float(width) ** 0.5},
           "layers": layers}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def moe_ff(experts, top, groups, keep, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top,
                       "groups": {"count": groups, "keep": keep}}}


def attention_layer(heads, kv_heads, dim, vdim, chunk, scale, mlp=None,
                    kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "mask": {"size": chunk}, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def rot(dims, base=10000.0, factor=None, original=None, fast=32.0,
        slow=1.0):
    r = {"dims": dims, "base": base}
    if factor:
        r["scaling"] = {"factor": factor, "original": original,
                        "fast": fast, "slow": slow}
    return r


def parallel_layer(heads, kv_heads, dim, vdim, scale, rotary, d_heads,
                   d_kv_heads, d_dim, d_vdim, conv, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale}
    if rotary:
        left["rot"] = rotary
    return {"type": "parallel",
            "mixer": {"left": left,
                      "right": {"heads": d_heads, "kv_heads": d_kv_heads,
                                "dim": d_dim, "vdim": d_vdim, "conv": conv}},
            "mlp": mlp}
