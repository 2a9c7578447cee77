"""Engine configuration: model architectures, cache sizing, scheduler knobs.

The reference gateway has no engine; these configs define the
net-new local provider models named by BASELINE.json: Llama-3 8B / 70B and
Mixtral 8x7B, plus tiny variants for CPU tests and smoke().
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional  # noqa: F401


@dataclass
class ModelConfig:
    name: str
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rope_base: float = 500000.0
    max_position: int = 8192
    norm_eps: float = 1e-5
    tie_embeddings: bool = False
    # Qwen2 family: bias on the fused qkv projection only (HF Qwen2
    # hardcodes q/k/v bias True, o/mlp bias False)
    qkv_bias: bool = False
    # HF rope_scaling dict (Llama-3.1 "llama3" wavelength-banded
    # rescale, or "linear"); None = plain RoPE
    rope_scaling: Optional[dict] = None
    # MoE (Mixtral): 0 experts => dense MLP
    num_experts: int = 0
    num_experts_per_tok: int = 2

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    def kv_bytes_per_token(self) -> int:
        # bf16 K + V per layer
        return 2 * self.num_kv_heads * self.head_dim * 2 * self.num_layers


# ---------------------------------------------------------------------------
# Fedatar: a per-layer hybrid decoder.  Every layer names its own mixer
# (a minGRU recurrence or windowed latent attention) and its own
# feed-forward (dense xIELU, relu^2 mixture of experts, or none), so the
# configuration is a LIST of layer specs instead of one set of sizes.
# ---------------------------------------------------------------------------
@dataclass
class RotarySpec:
    """Interleaved-pair rotary positions: pair i of the first `dims`
    entries turns by position * base**(-2i/dims)."""
    base: float = 10000.0
    dims: int = 0


@dataclass
class MinGRUSpec:
    width: int = 0


@dataclass
class LatentAttentionSpec:
    heads: int = 1
    dim: int = 64              # unrotated q/k entries per head
    rot_dim: int = 16          # rotated q/k entries per head (shared key)
    vdim: int = 64             # value entries per head
    kv_rank: int = 64          # cached latent width
    q_rank: int = 64           # query latent width
    scale: float = 0.0         # score multiplier; 0 => (dim+rot_dim)**-0.5
    window: int = 0            # keys seen per query incl. itself; 0 = all
    rot: RotarySpec = None

    def __post_init__(self):
        if self.rot is None:
            self.rot = RotarySpec(dims=self.rot_dim)
        if not self.scale:
            self.scale = float(self.dim + self.rot_dim) ** -0.5

    @property
    def cache_width(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass
class DenseFFSpec:
    ff: int = 0


@dataclass
class MoEFFSpec:
    experts: int = 1
    top: int = 1
    expert_ff: int = 0
    shared_ff: int = 0         # 0 => no always-on shared expert


@dataclass
class LayerSpec:
    type: str                  # "mingru" | "latent_attention"
    mixer: object              # MinGRUSpec | LatentAttentionSpec
    mlp: object = None         # DenseFFSpec | MoEFFSpec | None


@dataclass
class FedatarConfig:
    name: str
    hidden_size: int
    vocab_size: int
    layers: list
    norm_eps: float = 1e-5
    max_position: int = 1 << 20     # angles are computed, not tabulated
    architecture: str = "Fedatar"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(l.mlp, MoEFFSpec) for l in self.layers)

    def kv_bytes_per_token(self, itemsize: int = 2) -> int:
        """Paged bytes per token: only latent-attention layers page
        anything (latent + shared rotated key); minGRU layers hold one
        fixed-size state per sequence slot instead."""
        return max(itemsize, sum(
            l.mixer.cache_width * itemsize for l in self.layers
            if l.type == "latent_attention"))

    @staticmethod
    def from_dict(cfg: dict, name: str = "fedatar",
                  shapes: Optional[dict] = None) -> "FedatarConfig":
        """Parse the design's config.json.  `shapes` (tensor name ->
        shape, from the checkpoint header) fills sizes that the json
        leaves to the tensors."""
        shapes = shapes or {}
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m = l.get("mixer") or {}
            if l["type"] == "mingru":
                width = m.get("width")
                if width is None:
                    width = shapes[f"l{i}.mix.z"][0]
                mixer = MinGRUSpec(width=int(width))
            elif l["type"] == "latent_attention":
                rot = m.get("rot") or {}
                rot_dim = int(m["rot_dim"])
                q_rank = m.get("q_rank")
                if q_rank is None:
                    q_rank = shapes[f"l{i}.mix.dq"][0]
                mixer = LatentAttentionSpec(
                    heads=int(m["heads"]), dim=int(m["dim"]),
                    rot_dim=rot_dim, vdim=int(m["vdim"]),
                    kv_rank=int(m["kv_rank"]), q_rank=int(q_rank),
                    scale=float(m.get("scale") or 0.0),
                    window=int((m.get("mask") or {}).get("size") or 0),
                    rot=RotarySpec(base=float(rot.get("base", 10000.0)),
                                   dims=int(rot.get("dims", rot_dim))))
            else:
                raise ValueError(f"layer {i}: unknown mixer {l['type']!r}")
            f = l.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = DenseFFSpec(ff=int(f["ff"]))
            elif f["kind"] == "moe":
                sh = f.get("shared") or {}
                mlp = MoEFFSpec(experts=int(f["router"]["experts"]),
                                top=int(f["router"]["top"]),
                                expert_ff=int(f["expert"]["ff"]),
                                shared_ff=int(sh.get("ff") or 0))
            else:
                raise ValueError(f"layer {i}: unknown mlp {f['kind']!r}")
            layers.append(LayerSpec(type=l["type"], mixer=mixer, mlp=mlp))
        return FedatarConfig(
            name=name, hidden_size=int(cfg["width"]),
            vocab_size=int(cfg["vocab"]), layers=layers,
            norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-5)))


def fedatar_preset(name: str, width: int, vocab: int, pattern: str,
                   heads: int, dim: int, rot_dim: int, vdim: int,
                   kv_rank: int, q_rank: int, window: int, ff: int,
                   experts: int, top: int, expert_ff: int, shared_ff: int,
                   rot_base: float = 10000.0) -> FedatarConfig:
    """Layer pattern string: one letter pair per layer — mixer `g`
    (minGRU) or `a` (latent attention), then feed-forward `d` (dense),
    `m` (mixture) or `-` (none); e.g. "gd am gm"."""
    layers = []
    for tok in pattern.split():
        if tok[0] == "g":
            mixer, typ = MinGRUSpec(width=width), "mingru"
        else:
            mixer, typ = LatentAttentionSpec(
                heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                kv_rank=kv_rank, q_rank=q_rank, window=window,
                rot=RotarySpec(base=rot_base, dims=rot_dim)), \
                "latent_attention"
        mlp = {"d": DenseFFSpec(ff=ff),
               "m": MoEFFSpec(experts=experts, top=top,
                              expert_ff=expert_ff, shared_ff=shared_ff),
               "-": None}[tok[1]]
        layers.append(LayerSpec(type=typ, mixer=mixer, mlp=mlp))
    return FedatarConfig(name=name, hidden_size=width, vocab_size=vocab,
                         layers=layers)


# ---------------------------------------------------------------------------
# Mekevik: parallel-block decoder (mixer and feed-forward read the same
# residual through two norms and are added together) whose mixer is
# windowed SIGMOID attention: per-key logistic weights instead of a
# softmax, a learned bias per (distance bucket, head), weights mixed
# across heads, grouped key/value heads with their own value width,
# optional blending of every layer's values with the first layer's, and a
# sigmoid output gate.  Feed-forwards: a clamped gated unit or routed
# SwiGLU experts chosen by a softmax router.
# ---------------------------------------------------------------------------
def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of a distance-bias table for a key n tokens back: distances
    below rows/2 have a row each; beyond that rows are spaced
    logarithmically and the last one is reached at distance `far`."""
    import math

    half = rows // 2
    if n < half:
        return n
    if half == 0 or far <= half:
        # no logarithmic range to spread over: everything past the
        # exact rows shares the last one
        return rows - 1
    step = math.log(n / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


@dataclass
class SigmoidAttentionSpec:
    heads: int = 1
    kv_heads: int = 1          # query head h reads kv head h // (H/G)
    dim: int = 64              # query/key entries per head
    vdim: int = 64             # value entries per head
    scale: float = 0.0         # score multiplier; 0 => dim**-0.5
    window: int = 0            # keys seen per query incl. itself; 0 = all
    bias_rows: int = 32        # rows of the distance-bias table
    bias_far: float = 128.0    # distance that reaches the last row
    v_mix: bool = False        # blend values with the first such layer's

    def __post_init__(self):
        if not self.scale:
            self.scale = float(self.dim) ** -0.5
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")

    def bias_distances(self) -> int:
        """Distances that need their own entry when the bucket table is
        expanded per distance: everything from `bias_far` on shares the
        last row, and a window never looks further than itself."""
        import math

        n = int(math.ceil(self.bias_far)) + 1
        n = max(n, self.bias_rows // 2 + 1)
        return min(n, self.window) if self.window > 0 else n


@dataclass
class ClampedGLUSpec:
    ff: int = 0
    limit: float = 7.0         # gate clamped above, linear part both sides


@dataclass
class RoutedGLUSpec:
    experts: int = 1
    top: int = 1
    expert_ff: int = 0
    scale: float = 1.0         # multiplies the renormalised top-k weights


@dataclass
class MekevikConfig:
    name: str
    hidden_size: int
    vocab_size: int
    layers: list               # LayerSpec(type="attention", ...)
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    max_position: int = 1 << 20     # no position table anywhere
    architecture: str = "Mekevik"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(l.mlp, RoutedGLUSpec) for l in self.layers)

    def kv_bytes_per_token(self, itemsize: int = 2) -> int:
        return max(itemsize, sum(
            l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim) * itemsize
            for l in self.layers))

    @staticmethod
    def from_dict(cfg: dict, name: str = "mekevik",
                  shapes: Optional[dict] = None) -> "MekevikConfig":
        """Parse the design's config.json.  `shapes` (tensor name ->
        shape, from the checkpoint header) gives the sizes the json
        leaves to the tensors (rows of each distance-bias table)."""
        shapes = shapes or {}
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m = l.get("mixer") or {}
            if l["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer {l['type']!r}")
            rel = shapes.get(f"l{i}.mix.rel")
            mixer = SigmoidAttentionSpec(
                heads=int(m["heads"]),
                kv_heads=int(m.get("kv_heads") or m["heads"]),
                dim=int(m["dim"]), vdim=int(m.get("vdim") or m["dim"]),
                scale=float(m.get("scale") or 0.0),
                window=int((m.get("mask") or {}).get("size") or 0),
                bias_rows=int(rel[0]) if rel else int(
                    m.get("bias_rows", 32)),
                bias_far=float(m["bias_max"]),
                v_mix=bool(m.get("v_mix")))
            f = l.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = ClampedGLUSpec(ff=int(f["ff"]),
                                     limit=float(f["limit"]))
            elif f["kind"] == "moe":
                r = f["router"]
                mlp = RoutedGLUSpec(experts=int(r["experts"]),
                                    top=int(r["top"]),
                                    expert_ff=int(f["expert"]["ff"]),
                                    scale=float(r.get("scale", 1.0)))
            else:
                raise ValueError(f"layer {i}: unknown mlp {f['kind']!r}")
            layers.append(LayerSpec(type="attention", mixer=mixer, mlp=mlp))
        return MekevikConfig(
            name=name, hidden_size=int(cfg["width"]),
            vocab_size=int(cfg["vocab"]), layers=layers,
            norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-6)),
            embed_scale=float((cfg.get("embedding") or {}).get("scale",
                                                               1.0)),
            logit_scale=float(cfg.get("logit_scale", 1.0)))


def mekevik_preset(name: str, width: int, vocab: int, pattern: str,
                   heads: int, kv_heads: int, dim: int, vdim: int,
                   window: int, ff: int, experts: int, top: int,
                   expert_ff: int, bias_rows: int = 32,
                   bias_far: float = 128.0, limit: float = 7.0,
                   router_scale: float = 1.0, v_mix: bool = True,
                   embed_scale: float = 1.0, logit_scale: float = 1.0
                   ) -> MekevikConfig:
    """Layer pattern string: one letter per layer for its feed-forward —
    `d` (clamped dense unit), `m` (routed experts) or `-` (none)."""
    layers = []
    for tok in pattern.split():
        mixer = SigmoidAttentionSpec(
            heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
            window=window, bias_rows=bias_rows, bias_far=bias_far,
            v_mix=v_mix)
        mlp = {"d": ClampedGLUSpec(ff=ff, limit=limit),
               "m": RoutedGLUSpec(experts=experts, top=top,
                                  expert_ff=expert_ff, scale=router_scale),
               "-": None}[tok]
        layers.append(LayerSpec(type="attention", mixer=mixer, mlp=mlp))
    return MekevikConfig(name=name, hidden_size=width, vocab_size=vocab,
                         layers=layers, embed_scale=embed_scale,
                         logit_scale=logit_scale)


# ---------------------------------------------------------------------------
# Feditar: a per-layer decoder of RECURRENT mixers on an fp32 residual
# stream.  The embedding adds a hashed (previous, current) token-pair row
# and a learned position row; every layer is pre-norm (RMS, weight stored
# around zero) around one mixer and an optional relu^2 feed-forward.
# Mixers: an mLSTM matrix memory, a Mamba-2 state-space layer, or a
# PARALLEL pair — causal softmax attention (short convolutions on q/k/v,
# position-dependent query stretch, tanh score cap) beside an RWKV-style
# decayed outer-product memory — whose normed outputs are averaged.
# ---------------------------------------------------------------------------
@dataclass
class PairHashSpec:
    """Row of the pair table for (previous, current):
    (prev * mul_prev + cur * mul_cur) mod buckets; a sequence's first
    token takes row `buckets` (the table has buckets + 1 rows)."""
    buckets: int = 1
    mul_prev: int = 1
    mul_cur: int = 1


@dataclass
class MLSTMSpec:
    heads: int = 1
    dim: int = 64              # query/key entries per head
    vdim: int = 64             # value entries per head
    gate_cap: float = 15.0     # gates pass through cap * tanh(. / cap)


@dataclass
class Mamba2Spec:
    heads: int = 1
    vdim: int = 64             # channels per head (inner = heads * vdim)
    state: int = 64            # state entries per channel
    groups: int = 1            # B / C groups shared by heads
    conv: int = 4              # taps of the short convolution
    norm_groups: int = 1       # equal parts of the gated output norm

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class SoftcapAttentionSpec:
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64
    vdim: int = 64
    scale: float = 0.0         # 0 => dim ** -0.5
    softcap: float = 0.0       # 0 => scores are not squashed
    conv: int = 1              # taps of the q/k/v convolutions; 1 = none
    temp_coef: float = 0.0     # query *= 1 + coef * ln(floor((p+1)/every)+1)
    temp_every: int = 1

    def __post_init__(self):
        if not self.scale:
            self.scale = float(self.dim) ** -0.5


@dataclass
class DecayMemorySpec:
    """RWKV-style time mixing: per-channel decays from a low-rank map."""
    heads: int = 1
    dim: int = 64              # key = value entries per head
    decay_rank: int = 16


@dataclass
class ParallelMixerSpec:
    left: SoftcapAttentionSpec = None
    right: DecayMemorySpec = None


@dataclass
class Relu2FFSpec:
    ff: int = 0


@dataclass
class FeditarConfig:
    name: str
    hidden_size: int
    vocab_size: int
    layers: list               # LayerSpec(type="mlstm"|"mamba2"|"parallel")
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    pair_hash: PairHashSpec = None
    max_position: int = 2048   # rows of the learned position table
    architecture: str = "Feditar"

    def __post_init__(self):
        if self.pair_hash is None:
            self.pair_hash = PairHashSpec()

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return False

    def kv_bytes_per_token(self, itemsize: int = 2) -> int:
        """Paged bytes per token: only the attention half of a parallel
        mixer pages anything; everything else is fixed per slot."""
        return max(itemsize, sum(
            l.mixer.left.kv_heads * (l.mixer.left.dim + l.mixer.left.vdim)
            * itemsize for l in self.layers if l.type == "parallel"))

    @staticmethod
    def from_dict(cfg: dict, name: str = "feditar",
                  shapes: Optional[dict] = None) -> "FeditarConfig":
        """Parse the design's config.json.  `shapes` (tensor name ->
        shape, from the checkpoint header) gives what the json leaves
        to the tensors (rank of the decay map)."""
        shapes = shapes or {}
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m = l.get("mixer") or {}
            t = l["type"]
            if t == "mlstm":
                mixer = MLSTMSpec(heads=int(m["heads"]), dim=int(m["dim"]),
                                  vdim=int(m.get("vdim") or m["dim"]),
                                  gate_cap=float(m["gate_cap"]))
            elif t == "mamba2":
                mixer = Mamba2Spec(
                    heads=int(m["heads"]), vdim=int(m["vdim"]),
                    state=int(m["state"]), groups=int(m.get("groups") or 1),
                    conv=int(m["conv"]),
                    norm_groups=int(m.get("norm_groups") or 1))
            elif t == "parallel":
                a, b = m["left"], m["right"]
                qt = a.get("q_temp") or {}
                w1 = shapes.get(f"l{i}.mix.right.w1")
                mixer = ParallelMixerSpec(
                    left=SoftcapAttentionSpec(
                        heads=int(a["heads"]),
                        kv_heads=int(a.get("kv_heads") or a["heads"]),
                        dim=int(a["dim"]),
                        vdim=int(a.get("vdim") or a["dim"]),
                        scale=float(a.get("scale") or 0.0),
                        softcap=float(a.get("softcap") or 0.0),
                        conv=int(a.get("conv") or 1),
                        temp_coef=float(qt.get("coef") or 0.0),
                        temp_every=int(qt.get("every") or 1)),
                    right=DecayMemorySpec(
                        heads=int(b["heads"]), dim=int(b["dim"]),
                        decay_rank=int(w1[0]) if w1 else int(
                            b.get("decay_rank", 16))))
            else:
                raise ValueError(f"layer {i}: unknown mixer {t!r}")
            f = l.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = Relu2FFSpec(ff=int(f["ff"]))
            else:
                raise ValueError(f"layer {i}: unknown mlp {f['kind']!r}")
            layers.append(LayerSpec(type=t, mixer=mixer, mlp=mlp))
        e = cfg.get("embedding") or {}
        bg = e.get("bigram") or {}
        # table sizes the json leaves out come from the tensors
        pos_rows = cfg.get("max_positions") or (
            shapes["pos"][0] if "pos" in shapes else 2048)
        buckets = bg.get("buckets") or (
            shapes["bigram"][0] - 1 if "bigram" in shapes else 1)
        return FeditarConfig(
            name=name, hidden_size=int(cfg["width"]),
            vocab_size=int(cfg["vocab"]), layers=layers,
            norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-6)),
            embed_scale=float(e.get("scale", 1.0)),
            pair_hash=PairHashSpec(buckets=int(buckets),
                                   mul_prev=int(bg.get("mul_prev", 1)),
                                   mul_cur=int(bg.get("mul_cur", 1))),
            max_position=int(pos_rows))


def feditar_preset(name: str, width: int, vocab: int, pattern: str,
                   heads: int, dim: int, vdim: int, kv_heads: int = 0,
                   state: int = 64, groups: int = 1, ff: int = 0,
                   conv: int = 4, norm_groups: int = 1,
                   decay_rank: int = 32, gate_cap: float = 15.0,
                   softcap: float = 50.0, temp_coef: float = 0.1,
                   temp_every: int = 128, buckets: int = 4093,
                   max_position: int = 4096) -> FeditarConfig:
    """Layer pattern string: one letter pair per layer — mixer `x`
    (mLSTM), `s` (Mamba-2) or `p` (parallel attention + decayed
    memory), then feed-forward `d` (relu^2) or `-` (none); e.g.
    "x- s- pd"."""
    layers = []
    for tok in pattern.split():
        if tok[0] == "x":
            typ, mixer = "mlstm", MLSTMSpec(heads=heads, dim=dim, vdim=vdim,
                                            gate_cap=gate_cap)
        elif tok[0] == "s":
            typ, mixer = "mamba2", Mamba2Spec(
                heads=heads, vdim=vdim, state=state, groups=groups,
                conv=conv, norm_groups=norm_groups)
        else:
            typ, mixer = "parallel", ParallelMixerSpec(
                left=SoftcapAttentionSpec(
                    heads=heads, kv_heads=kv_heads or heads, dim=dim,
                    vdim=vdim, softcap=softcap, conv=conv,
                    temp_coef=temp_coef, temp_every=temp_every),
                right=DecayMemorySpec(heads=heads, dim=dim,
                                      decay_rank=decay_rank))
        mlp = Relu2FFSpec(ff=ff) if tok[1] == "d" else None
        layers.append(LayerSpec(type=typ, mixer=mixer, mlp=mlp))
    return FeditarConfig(
        name=name, hidden_size=width, vocab_size=vocab, layers=layers,
        embed_scale=float(width) ** 0.5,
        pair_hash=PairHashSpec(buckets=buckets, mul_prev=8191, mul_cur=131),
        max_position=max_position)


# ---------------------------------------------------------------------------
# Bozolorn: a per-layer decoder with sandwich norms (an RMS norm before
# AND after every sublayer), a small per-layer token embedding added after
# the feed-forward, and mixture-of-experts feed-forwards whose sigmoid
# router picks experts inside the best expert groups.  Mixers: softmax
# attention without rotation, with a linear distance bias, restricted to
# position chunks and gated at its output (a layer may borrow another
# layer's keys and values); or a PARALLEL pair of rotated softmax attention
# with a unit sink in its denominator beside a gated delta-rule memory.
# ---------------------------------------------------------------------------
@dataclass
class YarnRotarySpec:
    """Interleaved-pair rotary positions on the first `dims` entries of a
    head with YaRN frequency interpolation: with where(t) = dims *
    ln(original / (2 pi t)) / (2 ln base), lo = max(floor(where(fast)),
    0), hi = min(ceil(where(slow)), dims - 1) and ramp_i = clamp((i - lo)
    / max(hi - lo, 0.001), 0, 1), pair i turns by position * (f_i /
    factor * ramp_i + f_i * (1 - ramp_i)), f_i = base**(-2i/dims); cos
    and sin are multiplied by 0.1 ln(factor) + 1.  factor <= 0 or 1 with
    no `original` means plain rotation."""
    base: float = 10000.0
    dims: int = 0
    factor: float = 0.0        # 0 => no interpolation
    original: float = 0.0
    fast: float = 32.0
    slow: float = 1.0

    def frequencies(self):
        """([dims/2] angular steps as python floats, cos/sin factor)."""
        import math

        f = [self.base ** (-2.0 * i / self.dims)
             for i in range(self.dims // 2)]
        if not self.factor:
            return f, 1.0

        def where(turns):
            return self.dims * math.log(
                self.original / (2.0 * math.pi * turns)) / (
                    2.0 * math.log(self.base))

        lo = max(math.floor(where(self.fast)), 0)
        hi = min(math.ceil(where(self.slow)), self.dims - 1)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(fi / self.factor * ramp + fi * (1.0 - ramp))
        return out, 0.1 * math.log(self.factor) + 1.0


@dataclass
class ChunkBiasAttentionSpec:
    """Softmax attention without rotation: score = q.k * scale - slope_h
    * (i - j) with slope_h = 2**(-8 (h + 1) / heads); position i sees j
    <= i of its own chunk of `chunk` positions (0 = plain causal);
    sigmoid output gate.  kv_from = index of the layer whose keys and
    values this layer reads instead of projecting its own (-1 = own)."""
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64
    vdim: int = 64
    scale: float = 0.0         # 0 => dim ** -0.5
    chunk: int = 0
    kv_from: int = -1

    def __post_init__(self):
        if not self.scale:
            self.scale = float(self.dim) ** -0.5


@dataclass
class SinkAttentionSpec:
    """Causal softmax attention with projection biases, per-head RMS
    norm of queries and keys, partial rotary positions, and one more
    term of score 0 and no value in the softmax denominator."""
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64
    vdim: int = 64
    scale: float = 0.0         # 0 => dim ** -0.5
    rot: YarnRotarySpec = None  # None => no rotation

    def __post_init__(self):
        if not self.scale:
            self.scale = float(self.dim) ** -0.5


@dataclass
class DeltaRuleSpec:
    """Gated delta-rule memory: `kv_heads` query/key heads of `dim`
    entries shared by groups of the `heads` value heads of `vdim`
    entries; q, k, v pass a causal convolution of `conv` taps and silu."""
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64
    vdim: int = 64
    conv: int = 4

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim


@dataclass
class SinkDeltaPairSpec:
    left: SinkAttentionSpec = None
    right: DeltaRuleSpec = None


@dataclass
class GroupRoutedSpec:
    """Clamped gated experts chosen by a sigmoid router: choice score =
    sigmoid(logit) + correction; the experts form `groups` equal groups
    of neighbours, a group scores the sum of its two best choice scores,
    only experts of the best `keep` groups can be chosen; the `top`
    chosen experts are weighted by their plain sigmoid scores."""
    experts: int = 1
    top: int = 1
    groups: int = 1
    keep: int = 1
    expert_ff: int = 0
    limit: float = 7.0


@dataclass
class BozolornConfig:
    name: str
    hidden_size: int
    vocab_size: int
    layers: list               # LayerSpec(type="attention"|"parallel")
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    side_dim: int = 0          # per-layer token embedding width; 0 = none
    max_position: int = 1 << 20     # angles are computed, not tabulated
    architecture: str = "Bozolorn"

    def __post_init__(self):
        for i, l in enumerate(self.layers):
            if l.type != "attention" or l.mixer.kv_from < 0:
                continue
            src = l.mixer.kv_from
            if not (0 <= src < i) or self.layers[src].type != "attention" \
                    or self.layers[src].mixer.kv_from >= 0:
                raise ValueError(
                    f"layer {i}: kv_from must name an earlier attention "
                    "layer that projects its own keys and values")
            o = self.layers[src].mixer
            if (o.kv_heads, o.dim, o.vdim) != (
                    l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim):
                raise ValueError(
                    f"layer {i}: key/value sizes differ from layer {src}'s")

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(l.mlp is not None for l in self.layers)

    def kv_bytes_per_token(self, itemsize: int = 2) -> int:
        """Paged bytes per token: the attention layers that own keys and
        values and the attention half of every parallel mixer; the
        delta-rule memories are fixed per slot."""
        n = 0
        for l in self.layers:
            a = l.mixer.left if l.type == "parallel" else l.mixer
            if l.type == "parallel" or a.kv_from < 0:
                n += a.kv_heads * (a.dim + a.vdim) * itemsize
        return max(itemsize, n)

    @staticmethod
    def from_dict(cfg: dict, name: str = "bozolorn",
                  shapes: Optional[dict] = None) -> "BozolornConfig":
        """Parse the design's config.json (every size and constant is in
        it; `shapes` is accepted for symmetry with the other designs)."""

        def rotary(r):
            if not r:
                return None
            sc = r.get("scaling") or {}
            return YarnRotarySpec(
                base=float(r["base"]), dims=int(r["dims"]),
                factor=float(sc.get("factor") or 0.0),
                original=float(sc.get("original") or 0.0),
                fast=float(sc.get("fast", 32.0)),
                slow=float(sc.get("slow", 1.0)))

        def attention(m):
            kv_from = m.get("kv_from")
            return ChunkBiasAttentionSpec(
                heads=int(m["heads"]),
                kv_heads=int(m.get("kv_heads") or m["heads"]),
                dim=int(m["dim"]), vdim=int(m.get("vdim") or m["dim"]),
                scale=float(m.get("scale") or 0.0),
                chunk=int((m.get("mask") or {}).get("size") or 0),
                kv_from=-1 if kv_from is None else int(kv_from))

        layers = []
        for i, l in enumerate(cfg["layers"]):
            m = l.get("mixer") or {}
            t = l["type"]
            if t == "attention":
                mixer = attention(m)
            elif t == "parallel":
                a, b = m["left"], m["right"]
                mixer = SinkDeltaPairSpec(
                    left=SinkAttentionSpec(
                        heads=int(a["heads"]),
                        kv_heads=int(a.get("kv_heads") or a["heads"]),
                        dim=int(a["dim"]),
                        vdim=int(a.get("vdim") or a["dim"]),
                        scale=float(a.get("scale") or 0.0),
                        rot=rotary(a.get("rot"))),
                    right=DeltaRuleSpec(
                        heads=int(b["heads"]),
                        kv_heads=int(b.get("kv_heads") or b["heads"]),
                        dim=int(b["dim"]),
                        vdim=int(b.get("vdim") or b["dim"]),
                        conv=int(b.get("conv") or 1)))
            else:
                raise ValueError(f"layer {i}: unknown mixer {t!r}")
            f = l.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "moe":
                r = f["router"]
                gr = r.get("groups") or {}
                mlp = GroupRoutedSpec(
                    experts=int(r["experts"]), top=int(r["top"]),
                    groups=int(gr.get("count") or 1),
                    keep=int(gr.get("keep") or gr.get("count") or 1),
                    expert_ff=int(f["expert"]["ff"]),
                    limit=float(f["expert"]["limit"]))
                if mlp.experts % mlp.groups:
                    raise ValueError(
                        f"layer {i}: {mlp.experts} experts do not split "
                        f"into {mlp.groups} equal groups")
            else:
                raise ValueError(f"layer {i}: unknown mlp {f['kind']!r}")
            layers.append(LayerSpec(type=t, mixer=mixer, mlp=mlp))
        return BozolornConfig(
            name=name, hidden_size=int(cfg["width"]),
            vocab_size=int(cfg["vocab"]), layers=layers,
            norm_eps=float((cfg.get("norm") or {}).get("eps", 1e-6)),
            embed_scale=float((cfg.get("embedding") or {}).get("scale",
                                                               1.0)),
            side_dim=int((cfg.get("token_side") or {}).get("dim") or 0))


def bozolorn_preset(name: str, width: int, vocab: int, pattern: str,
                    heads: int, kv_heads: int, dim: int, vdim: int,
                    chunk: int, rot_dims: int, d_heads: int,
                    d_kv_heads: int, d_dim: int, d_vdim: int,
                    experts: int, top: int, groups: int, keep: int,
                    expert_ff: int, conv: int = 4, limit: float = 7.0,
                    side_dim: int = 0, rot_base: float = 1000000.0,
                    yarn_factor: float = 0.0,
                    yarn_original: float = 0.0) -> BozolornConfig:
    """Layer pattern string: one token per layer — mixer `a` (chunked
    attention), `a<j>` (the same, reading layer j's keys and values) or
    `p` (parallel sink attention + delta rule), then `m` (experts) or
    `-` (no feed-forward); e.g. "pm am pm a1m p-"."""
    layers = []
    for tok in pattern.split():
        if tok[0] == "a":
            typ, mixer = "attention", ChunkBiasAttentionSpec(
                heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                chunk=chunk, kv_from=int(tok[1:-1]) if tok[1:-1] else -1)
        else:
            typ, mixer = "parallel", SinkDeltaPairSpec(
                left=SinkAttentionSpec(
                    heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                    rot=YarnRotarySpec(base=rot_base, dims=rot_dims,
                                       factor=yarn_factor,
                                       original=yarn_original)
                    if rot_dims else None),
                right=DeltaRuleSpec(heads=d_heads, kv_heads=d_kv_heads,
                                    dim=d_dim, vdim=d_vdim, conv=conv))
        mlp = GroupRoutedSpec(experts=experts, top=top, groups=groups,
                              keep=keep, expert_ff=expert_ff,
                              limit=limit) if tok[-1] == "m" else None
        layers.append(LayerSpec(type=typ, mixer=mixer, mlp=mlp))
    return BozolornConfig(name=name, hidden_size=width, vocab_size=vocab,
                          layers=layers, embed_scale=float(width) ** 0.5,
                          side_dim=side_dim)


# Architectures from the public model cards (random-init weights — no network).
MODEL_PRESETS = {
    "llama-3-8b": ModelConfig(
        name="llama-3-8b",
        hidden_size=4096,
        num_layers=32,
        num_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=128256,
        rope_base=500000.0,
    ),
    "llama-3-70b": ModelConfig(
        name="llama-3-70b",
        hidden_size=8192,
        num_layers=80,
        num_heads=64,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=28672,
        vocab_size=128256,
        rope_base=500000.0,
    ),
    "llama-3.1-8b": ModelConfig(
        name="llama-3.1-8b",
        hidden_size=4096,
        num_layers=32,
        num_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=128256,
        rope_base=500000.0,
        max_position=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
    ),
    "llama-3.1-70b": ModelConfig(
        name="llama-3.1-70b",
        hidden_size=8192,
        num_layers=80,
        num_heads=64,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=28672,
        vocab_size=128256,
        rope_base=500000.0,
        max_position=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0,
                      "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 8192},
    ),
    "mixtral-8x7b": ModelConfig(
        name="mixtral-8x7b",
        hidden_size=4096,
        num_layers=32,
        num_heads=32,
        num_kv_heads=8,
        head_dim=128,
        intermediate_size=14336,
        vocab_size=32000,
        rope_base=1000000.0,
        num_experts=8,
        num_experts_per_tok=2,
    ),
    "qwen2.5-7b": ModelConfig(
        name="qwen2.5-7b",
        hidden_size=3584,
        num_layers=28,
        num_heads=28,
        num_kv_heads=4,
        head_dim=128,
        intermediate_size=18944,
        vocab_size=152064,
        rope_base=1000000.0,
        max_position=32768,
        norm_eps=1e-6,
        qkv_bias=True,
    ),
    # phi-3-MEDIUM, not mini: the MFMA attention kernels are tiled for
    # head_dim=128 (mini's 96 would fail the kernels' TORCH_CHECK on
    # GPU; engine init rejects non-128 head_dim on cuda devices)
    "phi-3-medium": ModelConfig(
        name="phi-3-medium",
        hidden_size=5120,
        num_layers=40,
        num_heads=40,
        num_kv_heads=10,
        head_dim=128,
        intermediate_size=17920,
        vocab_size=32064,
        rope_base=10000.0,
        max_position=4096,
    ),
    # tiny models for CPU tests / smoke
    "tiny-llama": ModelConfig(
        name="tiny-llama",
        hidden_size=512,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=1024,
        vocab_size=512,
        rope_base=10000.0,
        max_position=2048,
    ),
    "tiny-qwen2": ModelConfig(
        name="tiny-qwen2",
        hidden_size=512,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=1024,
        vocab_size=512,
        rope_base=10000.0,
        max_position=2048,
        qkv_bias=True,
        tie_embeddings=True,
    ),
    # tiny Fedatar for CPU tests / smoke: both mixers, all three
    # feed-forward kinds
    "tiny-fedatar": fedatar_preset(
        "tiny-fedatar", width=128, vocab=512, pattern="gd am gm a-",
        heads=2, dim=32, rot_dim=8, vdim=32, kv_rank=48, q_rank=40,
        window=24, ff=192, experts=6, top=2, expert_ff=48, shared_ff=64),
    # layer-shape benchmark points at Mixtral-8x7B's width (one layer
    # of each kind is enough to price the kernels; see bench.py)
    "fedatar-4k": fedatar_preset(
        "fedatar-4k", width=4096, vocab=32000,
        pattern="gd am gm am gm am gm am",
        heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=512,
        q_rank=1536, window=4096, ff=14336, experts=8, top=2,
        expert_ff=14336, shared_ff=0, rot_base=1000000.0),
    # tiny Mekevik for CPU tests / smoke: all three feed-forward kinds
    "tiny-mekevik": mekevik_preset(
        "tiny-mekevik", width=128, vocab=512, pattern="d m - m",
        heads=4, kv_heads=2, dim=24, vdim=16, window=20, ff=192,
        experts=6, top=2, expert_ff=48, bias_rows=12, bias_far=40.0,
        limit=1.5, router_scale=1.5, embed_scale=0.5, logit_scale=0.5),
    # layer-shape benchmark point at Mixtral-8x7B's width
    "mekevik-4k": mekevik_preset(
        "mekevik-4k", width=4096, vocab=32000, pattern="d m d m",
        heads=32, kv_heads=8, dim=128, vdim=128, window=4096, ff=14336,
        experts=8, top=2, expert_ff=14336, bias_rows=64, bias_far=4096.0),
    "tiny-feditar": feditar_preset(
        "tiny-feditar", width=96, vocab=320, pattern="x- s- pd s-",
        heads=4, kv_heads=2, dim=16, vdim=24, state=8, groups=2, ff=160,
        conv=3, norm_groups=2, decay_rank=8, gate_cap=8.0, softcap=20.0,
        temp_coef=0.25, temp_every=8, buckets=211, max_position=512),
    # layer-shape benchmark point at Llama-3-8B's width
    "feditar-4k": feditar_preset(
        "feditar-4k", width=4096, vocab=32000, pattern="x- s- pd pd",
        heads=32, kv_heads=8, dim=128, vdim=128, state=128, groups=8,
        ff=14336, norm_groups=8, decay_rank=64),
    # tiny Bozolorn for CPU tests / smoke: both mixers, a borrowed
    # key/value layer, a layer without feed-forward
    "tiny-bozolorn": bozolorn_preset(
        "tiny-bozolorn", width=96, vocab=320, pattern="pm am p- a1m",
        heads=4, kv_heads=2, dim=24, vdim=16, chunk=20, rot_dims=16,
        d_heads=4, d_kv_heads=2, d_dim=16, d_vdim=24, experts=6, top=2,
        groups=3, keep=2, expert_ff=40, conv=3, limit=1.5, side_dim=8,
        yarn_factor=4.0, yarn_original=64.0),
    # layer-shape benchmark point at Llama-3-8B's width
    "bozolorn-4k": bozolorn_preset(
        "bozolorn-4k", width=4096, vocab=32000, pattern="pm am pm a1m",
        heads=32, kv_heads=8, dim=128, vdim=128, chunk=1024, rot_dims=64,
        d_heads=32, d_kv_heads=8, d_dim=128, d_vdim=128, experts=8, top=2,
        groups=4, keep=2, expert_ff=14336, side_dim=64,
        yarn_factor=4.0, yarn_original=4096.0),
    "tiny-moe": ModelConfig(
        name="tiny-moe",
        hidden_size=512,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=128,
        intermediate_size=512,
        vocab_size=512,
        rope_base=10000.0,
        max_position=2048,
        num_experts=4,
        num_experts_per_tok=2,
    ),
}


@dataclass
class SamplingParams:
    max_new_tokens: int = 128
    temperature: float = 1.0
    top_k: int = 0          # <=0 disables
    top_p: float = 1.0      # >=1 disables
    stop_token_ids: tuple = ()
    ignore_eos: bool = False
    # OpenAI logprobs: -1 = off; >=0 = return the sampled token's logprob
    # plus that many top alternatives per step (capped at 20, like OpenAI)
    logprobs: int = -1
    # OpenAI seed: per-request deterministic sampling.  The per-seq tick
    # keeps counting across preemption/rebuild, so a seeded request is
    # reproducible even under KV pressure (tested). None = engine RNG.
    seed: Optional[int] = None
    # OpenAI repetition penalties (0 = off). Exact on the eager path; on
    # the async graph path the host's token view lags one step, so the
    # in-flight token's penalty is applied device-side (see sampler.py).
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    # OpenAI logit_bias: {token_id: bias in [-100, 100]} added to the
    # logits every step (None = off)
    logit_bias: Optional[dict] = None


@dataclass
class EngineConfig:
    model: ModelConfig
    block_size: int = 16
    num_gpu_blocks: Optional[int] = None   # None => size from free HBM
    gpu_memory_utilization: float = 0.90
    max_num_seqs: int = 256
    max_batched_tokens: int = 8192
    max_model_len: int = 8192
    use_hip_graphs: bool = True
    enforce_eager: bool = False
    # serving mode: capture every decode bucket at engine init so no
    # client ever pays a ~1 s first-capture stall mid-stream (the bench
    # path leaves this off — it uses one fixed bucket)
    capture_at_init: bool = False
    # prefix caching: hash-indexed reuse of full prompt blocks across
    # requests (suffix-only extend-prefill).  Opt-in.
    enable_prefix_caching: bool = False
    # chunked prefill: max_batched_tokens becomes a HARD budget — a long
    # prompt prefills in successive chunks (paged-extend attention) so a
    # burst never stalls in-flight decodes for a whole long prefill.
    enable_chunked_prefill: bool = False
    # strict admission priority: always prefill when prompts wait
    # (vLLM-style, TTFT-optimal under bursts) instead of alternating
    # prefill/decode rounds (ITL-optimal).  See scheduler.py.
    scheduler_prefill_first: bool = False
    # same-step mixed batches: a round with pending prompts carries the
    # (chunked) prefill segment AND every running decode row in one
    # forward — no whole-round ITL bubble (scheduler.py; the mixed
    # round runs eagerly, pure decode keeps the hipGraph)
    enable_mixed_batches: bool = False
    # real checkpoint: HF-format directory (config.json +
    # *.safetensors); None keeps the seed-derived synthetic init
    # (engine/weights.py — the no-network default)
    weights_path: Optional[str] = None
    # compute dtype: "bfloat16" (serving default) or "float32" (true
    # 32-bit everywhere; only architectures whose kernels are typed for
    # it accept this — see engine/models/registry.py)
    dtype: str = "bfloat16"
    tensor_parallel_size: int = 1
    seed: int = 0

    @staticmethod
    def tiny_llama(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-llama"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def tiny_moe(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-moe"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def tiny_fedatar(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-fedatar"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def tiny_mekevik(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-mekevik"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def tiny_feditar(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-feditar"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def tiny_bozolorn(**kw) -> "EngineConfig":
        defaults = dict(
            model=MODEL_PRESETS["tiny-bozolorn"],
            num_gpu_blocks=64,
            max_num_seqs=8,
            max_batched_tokens=2048,
            max_model_len=512,
            use_hip_graphs=False,
        )
        defaults.update(kw)
        return EngineConfig(**defaults)

    @staticmethod
    def for_model(name: str, **kw) -> "EngineConfig":
        return EngineConfig(model=MODEL_PRESETS[name], **kw)
