"""Real checkpoint loading: safetensors + HF config ingestion.

The reference gateway is stateless and has no checkpoints; SURVEY.md §5
names model-weight loading at engine start as the rebuild's
checkpoint/resume analog.  This loader maps a HuggingFace-format
directory (config.json + *.safetensors) onto the engine's fused,
TP-sharded parameter layout:

  model.embed_tokens.weight                  -> embed
  layers.N.self_attn.{q,k,v}_proj.weight     -> layer.attn.qkv   (fused,
                                                column-sharded per rank)
  layers.N.self_attn.qkv_proj.weight         -> same (HF Phi-3 ships the
                                                fusion pre-done; sections
                                                are sliced per rank)
  layers.N.mlp.gate_up_proj.weight           -> layer.mlp.gate_up (Phi-3)
  layers.N.self_attn.o_proj.weight           -> layer.attn.o_proj (row)
  layers.N.mlp.{gate,up}_proj.weight         -> layer.mlp.gate_up (fused)
  layers.N.mlp.down_proj.weight              -> layer.mlp.down_proj (row)
  layers.N.{input,post_attention}_layernorm  -> norms
  model.norm.weight / lm_head.weight         -> final_norm / lm_head
  Mixtral: block_sparse_moe.gate             -> router
           experts.E.{w1,w3}                 -> gate_up[E] (fused)
           experts.E.w2                      -> down[E]

Reads are per-rank sliced BEFORE materialization (safetensors
get_slice => only this rank's shard is read from disk/mmap), so a 70B
TP=8 rank reads ~17.5 GB, not 140 GB.  Synthetic seed-derived init
remains the no-network default (parallel/layers.py)."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, List

import torch

from ..parallel.comm import tp_rank, tp_world_size
from .config import ModelConfig


def model_config_from_hf(path: str, name: str = "hf-model"
                         ) -> ModelConfig:
    """Build a ModelConfig from a HuggingFace config.json."""
    cfg = json.loads((Path(path) / "config.json").read_text())
    num_experts = int(cfg.get("num_local_experts") or 0)
    mtype = cfg.get("model_type", name)
    # HF Qwen2 hardcodes qkv bias True and carries no attention_bias
    # field; Llama-family configs carry attention_bias (default False)
    qkv_bias = bool(cfg.get("attention_bias", mtype in ("qwen2",
                                                        "qwen2_moe")))
    rs = cfg.get("rope_scaling")
    if isinstance(rs, dict) and (rs.get("rope_type") or rs.get("type")) \
            in ("default", None):
        rs = None
    return ModelConfig(
        name=mtype,
        qkv_bias=qkv_bias,
        rope_scaling=rs if isinstance(rs, dict) else None,
        hidden_size=int(cfg["hidden_size"]),
        num_layers=int(cfg["num_hidden_layers"]),
        num_heads=int(cfg["num_attention_heads"]),
        num_kv_heads=int(cfg.get("num_key_value_heads",
                                 cfg["num_attention_heads"])),
        head_dim=int(cfg.get("head_dim") or (
            int(cfg["hidden_size"]) // int(cfg["num_attention_heads"]))),
        intermediate_size=int(cfg["intermediate_size"]),
        vocab_size=int(cfg["vocab_size"]),
        rope_base=float(cfg.get("rope_theta", 10000.0)),
        max_position=int(cfg.get("max_position_embeddings", 8192)),
        norm_eps=float(cfg.get("rms_norm_eps", 1e-5)),
        tie_embeddings=bool(cfg.get("tie_word_embeddings", False)),
        num_experts=num_experts,
        num_experts_per_tok=int(cfg.get("num_experts_per_tok", 2)),
    )


class _Shards:
    """Tensor-name -> (file, slice api) index over a checkpoint dir."""

    def __init__(self, path: str):
        from safetensors import safe_open

        self.files: List = []
        self.index: Dict[str, int] = {}
        for f in sorted(Path(path).glob("*.safetensors")):
            h = safe_open(str(f), framework="pt")
            i = len(self.files)
            self.files.append(h)
            for name in h.keys():
                self.index[name] = i

    def keys(self):
        return self.index.keys()

    def full(self, name: str) -> torch.Tensor:
        return self.files[self.index[name]].get_tensor(name)

    def rows(self, name: str, lo: int, hi: int) -> torch.Tensor:
        """Row slice [lo:hi] without materializing the full tensor."""
        return self.files[self.index[name]].get_slice(name)[lo:hi]

    def cols(self, name: str, lo: int, hi: int) -> torch.Tensor:
        return self.files[self.index[name]].get_slice(name)[:, lo:hi]


def _copy(param: torch.nn.Parameter, src: torch.Tensor, what: str) -> None:
    if param.shape != src.shape:
        raise ValueError(
            f"{what}: checkpoint shape {tuple(src.shape)} != engine "
            f"shape {tuple(param.shape)}")
    param.data.copy_(src.to(param.dtype))


def load_llama_weights(model, path: str) -> int:
    """Load HF Llama-family weights into LlamaForCausalLM (TP-sharded).
    Returns the number of engine parameters written."""
    sh = _Shards(path)
    cfg = model.cfg
    tp, rank = tp_world_size(), tp_rank()
    hd = cfg.head_dim
    nq, nkv = cfg.num_heads // tp, cfg.num_kv_heads // tp
    inter = cfg.intermediate_size // tp
    loaded = 0

    _copy(model.embed, sh.full("model.embed_tokens.weight"), "embed")
    loaded += 1
    # HF Phi-3 ships PRE-FUSED tensors (qkv_proj / gate_up_proj); the
    # sections inside still need per-rank slicing
    fused_ckpt = "model.layers.0.self_attn.qkv_proj.weight" in sh.index
    for i, layer in enumerate(model.layers):
        p = f"model.layers.{i}."
        if fused_ckpt:
            qkv_name = p + "self_attn.qkv_proj.weight"
            Q = cfg.num_heads * hd          # full q section rows
            K = cfg.num_kv_heads * hd
            q = sh.rows(qkv_name, rank * nq * hd, (rank + 1) * nq * hd)
            kk = sh.rows(qkv_name, Q + rank * nkv * hd,
                         Q + (rank + 1) * nkv * hd)
            v = sh.rows(qkv_name, Q + K + rank * nkv * hd,
                        Q + K + (rank + 1) * nkv * hd)
        else:
            q = sh.rows(p + "self_attn.q_proj.weight",
                        rank * nq * hd, (rank + 1) * nq * hd)
            kk = sh.rows(p + "self_attn.k_proj.weight",
                         rank * nkv * hd, (rank + 1) * nkv * hd)
            v = sh.rows(p + "self_attn.v_proj.weight",
                        rank * nkv * hd, (rank + 1) * nkv * hd)
        _copy(layer.attn.qkv, torch.cat([q, kk, v], 0), f"l{i}.qkv")
        has_bias = (p + "self_attn.q_proj.bias") in sh.index
        if layer.attn.qkv_b is not None:
            if not has_bias:
                raise ValueError(
                    f"l{i}: model expects qkv bias (qkv_bias=True) but "
                    "the checkpoint has no self_attn.*.bias tensors")
            qb = sh.rows(p + "self_attn.q_proj.bias",
                         rank * nq * hd, (rank + 1) * nq * hd)
            kb = sh.rows(p + "self_attn.k_proj.bias",
                         rank * nkv * hd, (rank + 1) * nkv * hd)
            vb = sh.rows(p + "self_attn.v_proj.bias",
                         rank * nkv * hd, (rank + 1) * nkv * hd)
            _copy(layer.attn.qkv_b, torch.cat([qb, kb, vb], 0),
                  f"l{i}.qkv_bias")
        elif has_bias:
            raise ValueError(
                f"l{i}: checkpoint carries self_attn.*.bias but the "
                "model config has qkv_bias=False — architecture mismatch")
        o = sh.cols(p + "self_attn.o_proj.weight",
                    rank * nq * hd, (rank + 1) * nq * hd)
        _copy(layer.attn.o_proj.weight, o, f"l{i}.o")
        if fused_ckpt:
            gu_name = p + "mlp.gate_up_proj.weight"
            I = cfg.intermediate_size       # full gate section rows
            g = sh.rows(gu_name, rank * inter, (rank + 1) * inter)
            u = sh.rows(gu_name, I + rank * inter, I + (rank + 1) * inter)
        else:
            g = sh.rows(p + "mlp.gate_proj.weight",
                        rank * inter, (rank + 1) * inter)
            u = sh.rows(p + "mlp.up_proj.weight",
                        rank * inter, (rank + 1) * inter)
        _copy(layer.mlp.gate_up, torch.cat([g, u], 0), f"l{i}.gate_up")
        d = sh.cols(p + "mlp.down_proj.weight",
                    rank * inter, (rank + 1) * inter)
        _copy(layer.mlp.down_proj.weight, d, f"l{i}.down")
        _copy(layer.input_norm_w, sh.full(p + "input_layernorm.weight"),
              f"l{i}.in_norm")
        _copy(layer.post_norm_w,
              sh.full(p + "post_attention_layernorm.weight"),
              f"l{i}.post_norm")
        loaded += 6
    _copy(model.final_norm_w, sh.full("model.norm.weight"), "final_norm")
    loaded += 1
    if model.lm_head is not None:
        name = ("lm_head.weight" if "lm_head.weight" in sh.index
                else "model.embed_tokens.weight")
        _copy(model.lm_head.weight, sh.full(name), "lm_head")
        loaded += 1
    return loaded


def load_mixtral_weights(model, path: str) -> int:
    """Load HF Mixtral weights (experts TP-sharded like the dense MLP)."""
    sh = _Shards(path)
    cfg = model.cfg
    tp, rank = tp_world_size(), tp_rank()
    hd = cfg.head_dim
    nq, nkv = cfg.num_heads // tp, cfg.num_kv_heads // tp
    shard = cfg.intermediate_size // tp
    loaded = 0

    _copy(model.embed, sh.full("model.embed_tokens.weight"), "embed")
    loaded += 1
    for i, layer in enumerate(model.layers):
        p = f"model.layers.{i}."
        q = sh.rows(p + "self_attn.q_proj.weight",
                    rank * nq * hd, (rank + 1) * nq * hd)
        kk = sh.rows(p + "self_attn.k_proj.weight",
                     rank * nkv * hd, (rank + 1) * nkv * hd)
        v = sh.rows(p + "self_attn.v_proj.weight",
                    rank * nkv * hd, (rank + 1) * nkv * hd)
        _copy(layer.attn.qkv, torch.cat([q, kk, v], 0), f"l{i}.qkv")
        o = sh.cols(p + "self_attn.o_proj.weight",
                    rank * nq * hd, (rank + 1) * nq * hd)
        _copy(layer.attn.o_proj.weight, o, f"l{i}.o")
        moe = layer.moe
        _copy(moe.router.weight,
              sh.full(p + "block_sparse_moe.gate.weight"), f"l{i}.gate")
        gus, downs = [], []
        for e in range(cfg.num_experts):
            ep = p + f"block_sparse_moe.experts.{e}."
            w1 = sh.rows(ep + "w1.weight", rank * shard,
                         (rank + 1) * shard)          # gate
            w3 = sh.rows(ep + "w3.weight", rank * shard,
                         (rank + 1) * shard)          # up
            w2 = sh.cols(ep + "w2.weight", rank * shard,
                         (rank + 1) * shard)          # down
            gus.append(torch.cat([w1, w3], 0))
            downs.append(w2)
        _copy(moe.gate_up, torch.stack(gus), f"l{i}.experts.gate_up")
        _copy(moe.down, torch.stack(downs), f"l{i}.experts.down")
        # keep the K-major bmm copies in sync (mixtral.py: contiguous-B
        # is both the hipBLASLt fault fix and faster)
        moe.gate_up_t.data.copy_(
            moe.gate_up.data.transpose(1, 2).contiguous())
        moe.down_t.data.copy_(moe.down.data.transpose(1, 2).contiguous())
        _copy(layer.input_norm_w, sh.full(p + "input_layernorm.weight"),
              f"l{i}.in_norm")
        _copy(layer.post_norm_w,
              sh.full(p + "post_attention_layernorm.weight"),
              f"l{i}.post_norm")
        loaded += 7
    _copy(model.final_norm_w, sh.full("model.norm.weight"), "final_norm")
    loaded += 1
    if model.lm_head is not None:
        _copy(model.lm_head.weight, sh.full("lm_head.weight"), "lm_head")
        loaded += 1
    return loaded


def load_fedatar_weights(model, path: str) -> int:
    """Load a Fedatar checkpoint: tensors `l<i>.norm1|norm2[.b]`,
    `l<i>.mix.*`, `l<i>.mlp.*`, `embed`, `final.norm[.b]`, `head`.  The
    engine's fused layouts are assembled here: z|x|g stacked for the
    minGRU input GEMM; query-latent | kv-latent+rotated-key | head-gate
    stacked for the attention down projection; per-head key/value
    up-projections reshaped for the absorbed batched GEMMs; experts
    stacked K-major.  Norm weights, sinks, activation constants and the
    router stay fp32."""
    from .config import DenseFFSpec, MoEFFSpec

    sh = _Shards(path)
    cfg = model.cfg
    n = 0

    def put(param, src, what):
        nonlocal n
        _copy(param, src, what)
        n += 1

    def norm(params, name):
        put(params.weight, sh.full(name), name)
        put(params.bias, sh.full(name + ".b"), name + ".b")

    put(model.embed, sh.full("embed"), "embed")
    for i, (spec, layer) in enumerate(zip(cfg.layers, model.layers)):
        p = f"l{i}."
        norm(layer.norm1, p + "norm1")
        mx, m = layer.mixer, p + "mix."
        if spec.type == "mingru":
            W = spec.mixer.width
            put(mx.zxg, torch.cat([sh.full(m + "z"), sh.full(m + "x"),
                                   sh.full(m + "g")], 0), m + "z|x|g")
            put(mx.zxg_b, torch.cat([
                sh.full(m + "z.b"), sh.full(m + "x.b"),
                torch.zeros(W, dtype=sh.full(m + "z.b").dtype)], 0),
                m + "z.b|x.b")
            put(mx.o, sh.full(m + "o"), m + "o")
        else:
            a = spec.mixer
            put(mx.down, torch.cat([sh.full(m + "dq"), sh.full(m + "dkv"),
                                    sh.full(m + "g")], 0), m + "dq|dkv|g")
            put(mx.qnorm_w, sh.full(m + "dq.norm"), m + "dq.norm")
            put(mx.kvnorm_w, sh.full(m + "dkv.norm"), m + "dkv.norm")
            put(mx.uq, sh.full(m + "uq"), m + "uq")
            put(mx.uk, sh.full(m + "uk").view(a.heads, a.dim, a.kv_rank),
                m + "uk")
            put(mx.uv_t, sh.full(m + "uv").view(
                a.heads, a.vdim, a.kv_rank).transpose(1, 2), m + "uv")
            put(mx.sink, sh.full(m + "sink"), m + "sink")
            put(mx.o, sh.full(m + "o"), m + "o")
        if spec.mlp is None:
            continue
        norm(layer.norm2, p + "norm2")
        f, ff = layer.mlp, p + "mlp."
        if isinstance(spec.mlp, DenseFFSpec):
            put(f.up, sh.full(ff + "up"), ff + "up")
            put(f.down, sh.full(ff + "down"), ff + "down")
            put(f.act, sh.full(ff + "act"), ff + "act")
        elif isinstance(spec.mlp, MoEFFSpec):
            put(f.router_w, sh.full(ff + "router"), ff + "router")
            put(f.router_b, sh.full(ff + "router.b"), ff + "router.b")
            E = spec.mlp.experts
            put(f.up_t, torch.stack(
                [sh.full(ff + f"e{e}.up").t() for e in range(E)]),
                ff + "e*.up")
            put(f.down_t, torch.stack(
                [sh.full(ff + f"e{e}.down").t() for e in range(E)]),
                ff + "e*.down")
            if f.shared_up is not None:
                put(f.shared_up, sh.full(ff + "shared.up"),
                    ff + "shared.up")
                put(f.shared_down, sh.full(ff + "shared.down"),
                    ff + "shared.down")
    norm(model.final_norm, "final.norm")
    put(model.head, sh.full("head"), "head")
    return n


def load_mekevik_weights(model, path: str) -> int:
    """Load a Mekevik checkpoint: tensors `embed`, `l<i>.norm1|norm2`,
    `l<i>.mix.{q,k,v,g,o,q.norm,k.norm,rel,pb,talk,vmix}`,
    `l<i>.mlp.{gate,up,down}` or `l<i>.mlp.router` and
    `l<i>.mlp.e<j>.{gate,up,down}`, `final.norm`, `head`.  The engine's
    fused layouts are assembled here: q|k|v|g stacked for the attention
    input GEMM, gate|up stacked for the dense unit, experts stacked
    K-major with gate|up side by side.  Norm weights, bias tables, the
    head-mixing matrix and the router stay fp32; the per-distance bias
    table is rebuilt from the loaded bucket table afterwards."""
    from .config import ClampedGLUSpec, RoutedGLUSpec

    sh = _Shards(path)
    cfg = model.cfg
    n = 0

    def put(param, src, what):
        nonlocal n
        _copy(param, src, what)
        n += 1

    put(model.embed, sh.full("embed"), "embed")
    for i, (spec, layer) in enumerate(zip(cfg.layers, model.layers)):
        p = f"l{i}."
        put(layer.norm1_w, sh.full(p + "norm1"), p + "norm1")
        mx, m = layer.mixer, p + "mix."
        put(mx.qkvg, torch.cat([sh.full(m + "q"), sh.full(m + "k"),
                                sh.full(m + "v"), sh.full(m + "g")], 0),
            m + "q|k|v|g")
        put(mx.qnorm_w, sh.full(m + "q.norm"), m + "q.norm")
        put(mx.knorm_w, sh.full(m + "k.norm"), m + "k.norm")
        put(mx.rel, sh.full(m + "rel"), m + "rel")
        put(mx.pb, sh.full(m + "pb"), m + "pb")
        put(mx.talk, sh.full(m + "talk"), m + "talk")
        put(mx.vmix, sh.full(m + "vmix").reshape(1), m + "vmix")
        put(mx.o, sh.full(m + "o"), m + "o")
        if spec.mlp is None:
            continue
        put(layer.norm2_w, sh.full(p + "norm2"), p + "norm2")
        f, ff = layer.mlp, p + "mlp."
        if isinstance(spec.mlp, ClampedGLUSpec):
            put(f.gate_up, torch.cat([sh.full(ff + "gate"),
                                      sh.full(ff + "up")], 0),
                ff + "gate|up")
            put(f.down, sh.full(ff + "down"), ff + "down")
        elif isinstance(spec.mlp, RoutedGLUSpec):
            put(f.router_w, sh.full(ff + "router"), ff + "router")
            E = spec.mlp.experts
            put(f.up_t, torch.stack([
                torch.cat([sh.full(ff + f"e{e}.gate"),
                           sh.full(ff + f"e{e}.up")], 0).t()
                for e in range(E)]), ff + "e*.gate|up")
            put(f.down_t, torch.stack(
                [sh.full(ff + f"e{e}.down").t() for e in range(E)]),
                ff + "e*.down")
    put(model.final_norm_w, sh.full("final.norm"), "final.norm")
    put(model.head, sh.full("head"), "head")
    model.rebuild_tables()
    return n


def load_feditar_weights(model, path: str) -> int:
    """Load a Feditar checkpoint: tensors `embed`, `bigram`, `pos`,
    `embed.norm`, `l<i>.norm1|norm2`, `l<i>.mix.*` per mixer kind,
    `l<i>.mlp.{up,down}`, `final.norm`.  The engine's layouts are
    assembled here: q|k|v|g stacked for the matrix memory's input GEMM
    and its two gate rows (with biases) kept apart in fp32; the
    state-space input projection split into its z|x|B|C rows and its
    fp32 step-size rows; q|k|v and their convolution filters stacked for
    the attention half of a parallel mixer; the decayed memory's four
    projections stacked K-major.  Norm weights stored around zero are
    held as 1 + w."""
    sh = _Shards(path)
    cfg = model.cfg
    n = 0

    def put(param, src, what):
        nonlocal n
        _copy(param, src, what)
        n += 1

    def one_plus(name):
        return 1.0 + sh.full(name).float()

    put(model.embed, sh.full("embed"), "embed")
    put(model.pair, sh.full("bigram"), "bigram")
    put(model.pos, sh.full("pos"), "pos")
    put(model.embed_norm_w, one_plus("embed.norm"), "embed.norm")
    for i, (spec, layer) in enumerate(zip(cfg.layers, model.layers)):
        p = f"l{i}."
        put(layer.norm1_w, one_plus(p + "norm1"), p + "norm1")
        mx, m = layer.mixer, p + "mix."
        if spec.type == "mlstm":
            put(mx.qkvg, torch.cat([sh.full(m + c) for c in "qkvg"], 0),
                m + "q|k|v|g")
            put(mx.gates_w, torch.cat([sh.full(m + "i"), sh.full(m + "f")],
                                      0), m + "i|f")
            put(mx.gates_b, torch.cat([sh.full(m + "i.b"),
                                       sh.full(m + "f.b")], 0), m + "i|f.b")
            put(mx.norm_w, sh.full(m + "norm"), m + "norm")
            put(mx.o, sh.full(m + "o"), m + "o")
        elif spec.type == "mamba2":
            rows = spec.mixer.inner + spec.mixer.conv_channels
            w_in = sh.full(m + "in")
            if w_in.shape[0] != rows + spec.mixer.heads:
                raise ValueError(
                    f"{m}in: checkpoint has {w_in.shape[0]} rows, the "
                    f"configuration needs {rows + spec.mixer.heads}")
            put(mx.in_main, w_in[:rows], m + "in[z|x|B|C]")
            put(mx.dt_w, w_in[rows:], m + "in[dt]")
            put(mx.dt_b, sh.full(m + "dt_bias"), m + "dt_bias")
            put(mx.conv_w, sh.full(m + "conv"), m + "conv")
            put(mx.conv_b, sh.full(m + "conv.b"), m + "conv.b")
            put(mx.a_log, sh.full(m + "A_log"), m + "A_log")
            put(mx.skip, sh.full(m + "D"), m + "D")
            put(mx.norm_w, sh.full(m + "norm"), m + "norm")
            put(mx.o, sh.full(m + "o"), m + "o")
        elif spec.type == "parallel":
            a, ml = mx.left, m + "left."
            put(a.qkv, torch.cat([sh.full(ml + c) for c in "qkv"], 0),
                ml + "q|k|v")
            if spec.mixer.left.conv > 1:
                put(a.conv_w, torch.cat(
                    [sh.full(ml + c + ".conv") for c in "qkv"], 0),
                    ml + "q|k|v.conv")
            put(a.o, sh.full(ml + "o"), ml + "o")
            b, mr = mx.right, m + "right."
            put(b.mu, torch.stack([sh.full(mr + "mu." + c)
                                   for c in b.MIXES]), mr + "mu.*")
            put(b.rkvg_t, torch.stack([sh.full(mr + c).t() for c in "rkvg"]),
                mr + "r|k|v|g")
            put(b.w1, sh.full(mr + "w1"), mr + "w1")
            put(b.w2, sh.full(mr + "w2"), mr + "w2")
            put(b.w0, sh.full(mr + "w0"), mr + "w0")
            put(b.bonus, sh.full(mr + "u"), mr + "u")
            put(b.norm_w, sh.full(mr + "norm"), mr + "norm")
            put(b.o, sh.full(mr + "o"), mr + "o")
            put(mx.left_out, sh.full(ml + "out"), ml + "out")
            put(mx.right_out, sh.full(mr + "out"), mr + "out")
        if spec.mlp is None:
            continue
        put(layer.norm2_w, one_plus(p + "norm2"), p + "norm2")
        put(layer.mlp.up, sh.full(p + "mlp.up"), p + "mlp.up")
        put(layer.mlp.down, sh.full(p + "mlp.down"), p + "mlp.down")
    put(model.final_norm_w, one_plus("final.norm"), "final.norm")
    return n


def load_bozolorn_weights(model, path: str) -> int:
    """Load a Bozolorn checkpoint: tensors `embed`, `side.embed`,
    `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.mix.*` per mixer kind,
    `l<i>.mlp.{router,correction}` and `l<i>.mlp.e<j>.{gate,up,down}`,
    `l<i>.side.{gate,proj,norm}`, `final.norm`, `head`.  The engine's
    layouts are assembled here: q|k|v|g (q|g for a layer that borrows its
    keys and values) stacked for the attention input GEMM; q|k|v with
    their biases for the rotated attention; q|k|v|g and the three
    convolution filters stacked for the delta-rule memory, its step and
    write-strength rows stacked apart in fp32 and its per-head norm
    weight repeated for every head; experts stacked K-major with gate|up
    side by side."""
    sh = _Shards(path)
    cfg = model.cfg
    n = 0

    def put(param, src, what):
        nonlocal n
        _copy(param, src, what)
        n += 1

    def cat(prefix, names, suffix=""):
        return torch.cat([sh.full(prefix + c + suffix) for c in names], 0)

    put(model.embed, sh.full("embed"), "embed")
    if model.side_embed is not None:
        put(model.side_embed, sh.full("side.embed"), "side.embed")
    for i, (spec, layer) in enumerate(zip(cfg.layers, model.layers)):
        p = f"l{i}."
        put(layer.norm1_w, sh.full(p + "norm1"), p + "norm1")
        put(layer.norm1b_w, sh.full(p + "norm1b"), p + "norm1b")
        mx, m = layer.mixer, p + "mix."
        if spec.type == "attention":
            rows = "qkvg" if mx.owns_kv else "qg"
            put(mx.qkvg, cat(m, rows), m + "|".join(rows))
            put(mx.o, sh.full(m + "o"), m + "o")
        else:
            a, ml = mx.left, m + "left."
            put(a.qkv, cat(ml, "qkv"), ml + "q|k|v")
            put(a.qkv_b, cat(ml, "qkv", ".b"), ml + "q|k|v.b")
            put(a.qnorm_w, sh.full(ml + "q.norm"), ml + "q.norm")
            put(a.knorm_w, sh.full(ml + "k.norm"), ml + "k.norm")
            put(a.o, sh.full(ml + "o"), ml + "o")
            b, mr = mx.right, m + "right."
            put(b.qkvg, cat(mr, "qkvg"), mr + "q|k|v|g")
            put(b.conv_w, cat(mr, "qkv", ".conv"), mr + "q|k|v.conv")
            put(b.ab_w, cat(mr, "ab"), mr + "a|b")
            put(b.a_log, sh.full(mr + "A_log"), mr + "A_log")
            put(b.dt_bias, sh.full(mr + "dt_bias"), mr + "dt_bias")
            put(b.norm_w, sh.full(mr + "norm").repeat(spec.mixer.right.heads),
                mr + "norm")
            put(b.o, sh.full(mr + "o"), mr + "o")
            put(mx.left_out, sh.full(ml + "out"), ml + "out")
            put(mx.right_out, sh.full(mr + "out"), mr + "out")
        if spec.mlp is not None:
            put(layer.norm2_w, sh.full(p + "norm2"), p + "norm2")
            put(layer.norm2b_w, sh.full(p + "norm2b"), p + "norm2b")
            f, ff = layer.mlp, p + "mlp."
            put(f.router_w, sh.full(ff + "router"), ff + "router")
            put(f.correction, sh.full(ff + "correction"), ff + "correction")
            E = spec.mlp.experts
            put(f.up_t, torch.stack([
                torch.cat([sh.full(ff + f"e{e}.gate"),
                           sh.full(ff + f"e{e}.up")], 0).t()
                for e in range(E)]), ff + "e*.gate|up")
            put(f.down_t, torch.stack(
                [sh.full(ff + f"e{e}.down").t() for e in range(E)]),
                ff + "e*.down")
        if layer.side is not None:
            sd = p + "side."
            put(layer.side.gate, sh.full(sd + "gate"), sd + "gate")
            put(layer.side.proj, sh.full(sd + "proj"), sd + "proj")
            put(layer.side.norm_w, sh.full(sd + "norm"), sd + "norm")
    put(model.final_norm_w, sh.full("final.norm"), "final.norm")
    put(model.head, sh.full("head"), "head")
    return n


def _is_gguf(path: str) -> bool:
    p = Path(path)
    if p.is_file():
        return p.suffix == ".gguf"
    # a directory with .gguf files and no safetensors is a GGUF
    # checkpoint (llama.cpp download layouts)
    return (not any(p.glob("*.safetensors"))
            and any(p.glob("*.gguf")))


def load_weights(model, path: str) -> int:
    """Dispatch on format (safetensors dir vs .gguf) and architecture;
    raises on shape/name mismatches (a checkpoint that does not match
    the configured architecture must fail loudly at startup, not
    generate garbage)."""
    if _is_gguf(path):
        from .gguf import load_gguf_weights

        return load_gguf_weights(model, path)
    if getattr(model.cfg, "architecture", "") == "Fedatar":
        return load_fedatar_weights(model, path)
    if getattr(model.cfg, "architecture", "") == "Mekevik":
        return load_mekevik_weights(model, path)
    if getattr(model.cfg, "architecture", "") == "Feditar":
        return load_feditar_weights(model, path)
    if getattr(model.cfg, "architecture", "") == "Bozolorn":
        return load_bozolorn_weights(model, path)
    if getattr(model.cfg, "is_moe", False):
        return load_mixtral_weights(model, path)
    return load_llama_weights(model, path)
