"""Plain float64 model of the Feditar design, token by token, one
function per mechanism.  It shares no code with the engine: weights come
in as a dict of numpy arrays under the checkpoint's tensor names, the
configuration as the parsed config.json dict.

Notation: D model width, T tokens of ONE sequence, H heads, G key/value
heads or groups, N key/state entries per head, P value entries per head.
"""
from __future__ import annotations

import math

import numpy as np


def rms_unit(x, eps):
    """x scaled to unit root mean square over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return np.logaddexp(0.0, x)


def logsigmoid(x):
    return -np.logaddexp(0.0, -x)


def embed(tokens, W, cfg, eps):
    """Scaled token row + hashed (previous, current) pair row + learned
    position row, then the one-plus norm."""
    e = cfg["embedding"]
    bg = e["bigram"]
    out = []
    for p, t in enumerate(tokens):
        x = W["embed"][t] * e["scale"]
        if p == 0:
            row = bg["buckets"]
        else:
            row = (tokens[p - 1] * bg["mul_prev"] + t * bg["mul_cur"]) \
                % bg["buckets"]
        x = x + W["bigram"][row] + W["pos"][p]
        out.append(norm_one_plus(x, W["embed.norm"], eps))
    return np.stack(out)


def short_conv(u, w, bias=None):
    """Per-channel causal filter: the LAST tap multiplies the current
    token, zeros before the sequence starts.  u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        acc = np.zeros(C) if bias is None else bias.copy()
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                acc = acc + w[:, j] * u[s]
        y[t] = acc
    return y


def softcap_attention(q, k, v, H, G, scale, cap, coef, every):
    """Causal softmax attention; grouped heads; the query is stretched
    by a slowly growing function of its position; scores are squashed
    through cap*tanh(./cap).  q [T, H, N], k [T, G, N], v [T, G, P]."""
    T = q.shape[0]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        temp = 1.0 + coef * math.log(math.floor((i + 1) / every) + 1.0)
        for h in range(H):
            g = h // (H // G)
            s = (k[: i + 1, g] @ (q[i, h] * temp)) * scale
            s = cap * np.tanh(s / cap)
            s = np.exp(s - s.max())
            out[i, h] = (s / s.sum()) @ v[: i + 1, g]
    return out


def left_mixer(h, W, pre, m):
    H, G, N, P = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q, k, v = (h @ W[pre + c].T for c in "qkv")
    if m.get("conv", 1) > 1:
        q = short_conv(q, W[pre + "q.conv"])
        k = short_conv(k, W[pre + "k.conv"])
        v = short_conv(v, W[pre + "v.conv"])
    o = softcap_attention(q.reshape(T, H, N), k.reshape(T, G, N),
                          v.reshape(T, G, P), H, G, m["scale"],
                          m["softcap"], m["q_temp"]["coef"],
                          m["q_temp"]["every"])
    return o.reshape(T, H * P) @ W[pre + "o"].T


def decayed_outer_scan(r, k, v, w, u):
    """Per head: o_t = (S + diag(u) k_t v_t^T)^T r_t, then
    S <- diag(w_t) S + k_t v_t^T.  All [T, H, N] (u [H, N])."""
    T, H, N = r.shape
    S = np.zeros((H, N, v.shape[2]))
    o = np.zeros_like(v)
    for t in range(T):
        for hd in range(H):
            kv = np.outer(k[t, hd], v[t, hd])
            o[t, hd] = (S[hd] + u[hd][:, None] * kv).T @ r[t, hd]
            S[hd] = w[t, hd][:, None] * S[hd] + kv
    return o


def right_mixer(h, W, pre, m, eps):
    H, N = m["heads"], m["dim"]
    T = h.shape[0]
    prev = np.concatenate([np.zeros((1, h.shape[1])), h[:-1]])
    mix = {s: h + (prev - h) * W[pre + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ W[pre + "r"].T).reshape(T, H, N)
    k = (mix["k"] @ W[pre + "k"].T).reshape(T, H, N)
    v = (mix["v"] @ W[pre + "v"].T).reshape(T, H, N)
    gate = silu(mix["g"] @ W[pre + "g"].T)
    lw = np.tanh(mix["w"] @ W[pre + "w1"].T) @ W[pre + "w2"].T \
        + W[pre + "w0"]
    w = np.exp(-np.exp(lw)).reshape(T, H, N)
    o = decayed_outer_scan(r, k, v, w, W[pre + "u"])
    o = rms_unit(o, eps).reshape(T, H * N)
    return (o * W[pre + "norm"] * gate) @ W[pre + "o"].T


def parallel_mixer(h, W, pre, m, eps):
    a = left_mixer(h, W, pre + "left.", m["left"])
    b = right_mixer(h, W, pre + "right.", m["right"], eps)
    return 0.5 * (rms_unit(a, eps) * W[pre + "left.out"]
                  + rms_unit(b, eps) * W[pre + "right.out"])


def mlstm_mixer(h, W, pre, m, eps):
    H, N, P, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).reshape(T, H, N) * N ** -0.5
    k = (h @ W[pre + "k"].T).reshape(T, H, N)
    v = (h @ W[pre + "v"].T).reshape(T, H, P)
    gi = cap * np.tanh((h @ W[pre + "i"].T + W[pre + "i.b"]) / cap)
    gf = logsigmoid(cap * np.tanh((h @ W[pre + "f"].T + W[pre + "f.b"])
                                  / cap))
    S = np.zeros((H, N, P))
    n = np.zeros((H, N))
    mx = np.zeros(H)
    o = np.zeros((T, H, P))
    for t in range(T):
        for hd in range(H):
            m_new = max(gf[t, hd] + mx[hd], gi[t, hd])
            a = math.exp(gf[t, hd] + mx[hd] - m_new)
            b = math.exp(gi[t, hd] - m_new)
            S[hd] = a * S[hd] + b * np.outer(k[t, hd], v[t, hd])
            n[hd] = a * n[hd] + b * k[t, hd]
            mx[hd] = m_new
            den = max(abs(n[hd] @ q[t, hd]), math.exp(-m_new)) + 1e-6
            o[t, hd] = S[hd].T @ q[t, hd] / den
    o = rms_unit(o, eps).reshape(T, H * P)
    return (o * W[pre + "norm"] * sigmoid(h @ W[pre + "g"].T)) \
        @ W[pre + "o"].T


def mamba2_mixer(h, W, pre, m, eps):
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ W[pre + "in"].T
    z = proj[:, :inner]
    xbc = proj[:, inner: 2 * inner + 2 * G * N]
    dt = softplus(proj[:, 2 * inner + 2 * G * N:] + W[pre + "dt_bias"])
    xbc = silu(short_conv(xbc, W[pre + "conv"], W[pre + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner: inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    S = np.zeros((H, N, P))
    y = np.zeros((T, H, P))
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            a = math.exp(-math.exp(W[pre + "A_log"][hd]) * dt[t, hd])
            S[hd] = a * S[hd] + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + W[pre + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms_unit(y.reshape(T, ng, inner // ng), eps).reshape(T, inner)
    return (y * W[pre + "norm"]) @ W[pre + "o"].T


def relu2_mlp(h, W, pre):
    a = np.maximum(h @ W[pre + "up"].T, 0.0)
    return (a * a) @ W[pre + "down"].T


def forward(W, cfg, tokens):
    """Returns (logits [T, vocab], residual after every layer
    [layers, T, D])."""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, W, cfg, eps)
    taps = []
    for i, l in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = norm_one_plus(x, W[pre + "norm1"], eps)
        if l["type"] == "parallel":
            d = parallel_mixer(h, W, pre + "mix.", l["mixer"], eps)
        elif l["type"] == "mlstm":
            d = mlstm_mixer(h, W, pre + "mix.", l["mixer"], eps)
        elif l["type"] == "mamba2":
            d = mamba2_mixer(h, W, pre + "mix.", l["mixer"], eps)
        else:
            raise ValueError(l["type"])
        x = x + d
        if l.get("mlp") is not None:
            x = x + relu2_mlp(norm_one_plus(x, W[pre + "norm2"], eps), W,
                              pre + "mlp.")
        taps.append(x.copy())
    logits = norm_one_plus(x, W["final.norm"], eps) @ W["embed"].T
    return logits, np.stack(taps)


# ---------------------------------------------------------------------------
# random checkpoints for the tests
# ---------------------------------------------------------------------------
def tensor_shapes(cfg):
    """Tensor name -> shape of a checkpoint of this configuration."""
    D, V = cfg["width"], cfg["vocab"]
    sh = {"embed": (V, D),
          "bigram": (cfg["embedding"]["bigram"]["buckets"] + 1, D),
          "pos": (cfg["max_positions"], D), "embed.norm": (D,),
          "final.norm": (D,)}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        sh[p + "norm1"] = (D,)
        if l["type"] == "mlstm":
            H, N, P = m["heads"], m["dim"], m["vdim"]
            sh.update({p + "mix.q": (H * N, D), p + "mix.k": (H * N, D),
                       p + "mix.v": (H * P, D), p + "mix.g": (H * P, D),
                       p + "mix.o": (D, H * P), p + "mix.norm": (H * P,),
                       p + "mix.i": (H, D), p + "mix.i.b": (H,),
                       p + "mix.f": (H, D), p + "mix.f.b": (H,)})
        elif l["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, cc = H * P, H * P + 2 * G * N
            sh.update({p + "mix.in": (inner + cc + H, D),
                       p + "mix.conv": (cc, m["conv"]),
                       p + "mix.conv.b": (cc,), p + "mix.dt_bias": (H,),
                       p + "mix.A_log": (H,), p + "mix.D": (H,),
                       p + "mix.norm": (inner,), p + "mix.o": (D, inner)})
        else:
            a, b = m["left"], m["right"]
            H, G, N, P = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            sh.update({q + "q": (H * N, D), q + "k": (G * N, D),
                       q + "v": (G * P, D), q + "o": (D, H * P),
                       q + "out": (D,)})
            if a["conv"] > 1:
                sh.update({q + "q.conv": (H * N, a["conv"]),
                           q + "k.conv": (G * N, a["conv"]),
                           q + "v.conv": (G * P, a["conv"])})
            r = p + "mix.right."
            HN = b["heads"] * b["dim"]
            R = b.get("decay_rank", 4)
            sh.update({r + "mu." + s: (D,) for s in "rkvgw"})
            sh.update({r + s: (HN, D) for s in "rkvg"})
            sh.update({r + "w1": (R, D), r + "w2": (HN, R), r + "w0": (HN,),
                       r + "u": (b["heads"], b["dim"]), r + "norm": (HN,),
                       r + "o": (D, HN), r + "out": (D,)})
        if l.get("mlp") is not None:
            sh.update({p + "norm2": (D,), p + "mlp.up": (l["mlp"]["ff"], D),
                       p + "mlp.down": (D, l["mlp"]["ff"])})
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
        if name in ("embed",):
            x = x * 0.5 / cfg["embedding"]["scale"]
        elif name in ("bigram", "pos"):
            x = x * 0.5
        elif last in ("norm1", "norm2") or name in ("embed.norm",
                                                    "final.norm"):
            x = x * 0.2                     # stored around zero
        elif last in ("norm", "out", "D"):
            x = 1.0 + x * 0.2
        elif ".mu." in name:
            x = torch.rand(shape, generator=g)
        elif last == "w0":
            x = -1.0 + x * 0.7
        elif last in ("A_log", "dt_bias", "u"):
            x = x * 0.5
        elif name.endswith("f.b"):
            x = 2.0 + x
        elif name.endswith("i.b") or name.endswith("conv.b"):
            x = x * 0.5
        elif last == "conv":
            x = x * 0.6
        elif len(shape) == 2:
            x = x * shape[1] ** -0.5 * (3.0 if last in ("i", "f", "w2")
                                        else 1.0)
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


def make_config(width, vocab, layers, buckets=97, mul_prev=7, mul_cur=3,
                scale=None, eps=1e-5, max_positions=700):
    return {"architecture": "Feditar", "width": width, "vocab": vocab,
            "max_positions": max_positions, "norm": {"eps": eps},
            "embedding": {"scale": scale or float(width) ** 0.5,
                          "bigram": {"buckets": buckets,
                                     "mul_prev": mul_prev,
                                     "mul_cur": mul_cur}},
            "layers": layers}


def mlstm_layer(heads, dim, vdim, cap=10.0, ff=0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim,
                                       "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mamba2_layer(heads, vdim, state, groups, conv, norm_groups, ff=0):
    return {"type": "mamba2",
            "mixer": {"heads": heads, "vdim": vdim, "state": state,
                      "groups": groups, "conv": conv,
                      "norm_groups": norm_groups},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def parallel_layer(heads, kv_heads, dim, vdim, conv, coef, every, scale,
                   softcap, r_heads, r_dim, ff=0):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads,
                               "dim": dim, "vdim": vdim, "conv": conv,
                               "q_temp": {"coef": coef, "every": every},
                               "scale": scale, "softcap": softcap},
                      "right": {"heads": r_heads, "dim": r_dim}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}
