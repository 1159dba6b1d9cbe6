"""Device-resident model weights in the layout the kernels stream: bf16,
q/k/v fused into one matrix and gate/up fused into one, every matrix re-tiled
once for the 16x16x32 MFMA (ops.tile_weights; layouts in include/sd_amd.h).
With fp8=True the layer matrices and the LM head are quantised at load to
fp8-e4m3 with one f32 scale per output row (weight-only: activations, norms,
biases and the embedding table stay bf16).

Sources: a Hugging Face style state dict (names as in transformers), a local
directory of *.safetensors shards, or seeded random initialisation.  The
reference only ever loads by hub name
(/root/reference/src/qwen_image_gen/model.py:46-65), which needs a network.
"""
from __future__ import annotations

import glob
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from . import ops
from .config import ModelConfig, rope_table


@dataclass
class LayerTensors:
    attn_norm_w: torch.Tensor
    qkv_w: "ops.TiledWeight"      # TILE_ROTARY
    o_w: "ops.TiledWeight"        # TILE_PLAIN
    mlp_norm_w: torch.Tensor
    up_w: "ops.TiledWeight"       # TILE_GATED (llama) / TILE_PLAIN (opt)
    down_w: "ops.TiledWeight"     # TILE_PLAIN
    attn_norm_b: Optional[torch.Tensor] = None
    qkv_b: Optional[torch.Tensor] = None
    o_b: Optional[torch.Tensor] = None
    mlp_norm_b: Optional[torch.Tensor] = None
    up_b: Optional[torch.Tensor] = None
    down_b: Optional[torch.Tensor] = None


@dataclass
class ModelWeights:
    cfg: ModelConfig
    embed: torch.Tensor           # row-major, or the tiled LM head's buffer when tied
    final_norm_w: torch.Tensor
    lm_head: "ops.TiledWeight"    # TILE_PLAIN
    layers: List[LayerTensors]
    embed_tiled: bool = False
    pos_table: Optional[torch.Tensor] = None
    final_norm_b: Optional[torch.Tensor] = None
    rope_cs: Optional[torch.Tensor] = None
    fp8: bool = False
    # LM head over a subset of the vocabulary (a draft model's cheaper head): head_map[i] is the
    # token id of head row i (int32, on the device); None = the whole vocabulary in order
    head_map: Optional[torch.Tensor] = None

    def nbytes(self) -> int:
        seen, total = set(), 0
        for t in self.tensors():
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    def tensors(self):
        def parts(t):
            if isinstance(t, ops.TiledWeight):
                yield t.data
                if t.scale is not None:
                    yield t.scale
            elif t is not None:
                yield t

        for t in (self.embed, self.final_norm_w, self.lm_head, self.pos_table, self.final_norm_b):
            yield from parts(t)
        for l in self.layers:
            for t in vars(l).values():
                yield from parts(t)


def _dev(t: torch.Tensor, device) -> torch.Tensor:
    return t.to(device=device, dtype=torch.bfloat16).contiguous()


def _tile_matrix(w: torch.Tensor, mode: int = ops.TILE_PLAIN, head_dim: int = 0,
                 fp8: bool = False) -> "ops.TiledWeight":
    if fp8:
        q, scale = ops.quantize_fp8(w)
        return ops.tile_weights(q, mode, head_dim, scale=scale)
    return ops.tile_weights(w, mode, head_dim)


def _head_subset(cfg: ModelConfig, head_subset, device):
    """(config whose head has one row per listed token, the ids as a device tensor)."""
    ids = torch.as_tensor(list(head_subset), dtype=torch.int64)
    if ids.numel() == 0 or ids.numel() % 16 or ids.min() < 0 or ids.max() >= cfg.vocab:
        raise ValueError("head_subset: a positive multiple of 16 token ids inside the vocabulary")
    if ids.unique().numel() != ids.numel():
        raise ValueError("head_subset: token ids must be distinct")
    if cfg.lm_vocab:
        raise ValueError("head_subset: the head is already a slice (vocabulary-parallel)")
    import dataclasses
    return dataclasses.replace(cfg, lm_vocab=int(ids.numel())), ids.to(device)


def _embed_and_head(embed: torch.Tensor, head, device, fp8: bool = False, subset=None):
    """Untied: row-major embedding + tiled head.  Tied: ONE tiled buffer serves
    both (the embedding gather reads rows out of the tiled layout); with fp8 the
    head is a quantised copy and the embedding table stays row-major bf16.  subset (token
    ids): the head keeps those rows only, in that order; the embedding table stays whole."""
    if subset is not None:
        src = embed if head is None else _dev(head, device)
        return embed, _tile_matrix(src[subset].contiguous(), fp8=fp8), False
    if head is None:
        if fp8:
            return embed, _tile_matrix(embed, fp8=True), False
        t = _tile_matrix(embed)
        return t.data, t, True
    return embed, _tile_matrix(_dev(head, device), fp8=fp8), False


def language_model_state(state: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The language model's tensors of a Qwen2-VL style checkpoint under the names of a text
    checkpoint: "model.language_model.X" -> "model.X", the vision tower ("visual.",
    "model.visual.") dropped.  Text checkpoints pass through unchanged."""
    out = {}
    for name, t in state.items():
        if name.startswith(("visual.", "model.visual.")):
            continue
        if name.startswith("model.language_model."):
            name = "model." + name[len("model.language_model."):]
        out[name] = t
    return out


def from_state_dict(cfg: ModelConfig, state: Dict[str, torch.Tensor], device="cuda",
                    fp8: bool = False, head_subset=None) -> ModelWeights:
    """head_subset (token ids, a multiple of 16 of them): the LM head computes logits for those
    tokens only (ModelWeights.head_map; for draft models: a head over the frequent tokens costs
    a fraction of the whole one, and whatever the draft cannot propose the target still emits)."""
    cfg.validate()
    state = language_model_state(state)
    sub = None
    if head_subset is not None:
        cfg, sub = _head_subset(cfg, head_subset, device)

    def _tile(w, mode=ops.TILE_PLAIN, head_dim=0):  # every layer matrix alike
        return _tile_matrix(w, mode, head_dim, fp8=fp8)

    g = lambda n: state[n]
    opt = lambda n: state.get(n)
    layers = []
    if cfg.arch == "llama":
        pre = "model."
        for i in range(cfg.n_layers):
            lp = f"{pre}layers.{i}."
            qkv_w = torch.cat([g(lp + "self_attn.q_proj.weight"), g(lp + "self_attn.k_proj.weight"),
                               g(lp + "self_attn.v_proj.weight")], dim=0)
            qb = opt(lp + "self_attn.q_proj.bias")
            qkv_b = None if qb is None else torch.cat(
                [qb, g(lp + "self_attn.k_proj.bias"), g(lp + "self_attn.v_proj.bias")], dim=0)
            up_w = torch.cat([g(lp + "mlp.gate_proj.weight"), g(lp + "mlp.up_proj.weight")], dim=0)
            layers.append(LayerTensors(
                attn_norm_w=_dev(g(lp + "input_layernorm.weight"), device),
                qkv_w=_tile(_dev(qkv_w, device), ops.TILE_ROTARY, cfg.head_dim),
                qkv_b=None if qkv_b is None else _dev(qkv_b, device),
                o_w=_tile(_dev(g(lp + "self_attn.o_proj.weight"), device)),
                mlp_norm_w=_dev(g(lp + "post_attention_layernorm.weight"), device),
                up_w=_tile(_dev(up_w, device), ops.TILE_GATED),
                down_w=_tile(_dev(g(lp + "mlp.down_proj.weight"), device))))
        embed, lm_head, tied = _embed_and_head(_dev(g(pre + "embed_tokens.weight"), device),
                                               opt("lm_head.weight"), device, fp8, sub)
        return ModelWeights(cfg=cfg, embed=embed, embed_tiled=tied, fp8=fp8,
                            final_norm_w=_dev(g(pre + "norm.weight"), device), lm_head=lm_head,
                            layers=layers, rope_cs=rope_table(cfg, device),
                            head_map=None if sub is None else sub.to(torch.int32))
    pre = "model.decoder."
    for i in range(cfg.n_layers):
        lp = f"{pre}layers.{i}."
        qkv_w = torch.cat([g(lp + f"self_attn.{n}_proj.weight") for n in "qkv"], dim=0)
        qkv_b = torch.cat([g(lp + f"self_attn.{n}_proj.bias") for n in "qkv"], dim=0)
        layers.append(LayerTensors(
            attn_norm_w=_dev(g(lp + "self_attn_layer_norm.weight"), device),
            attn_norm_b=_dev(g(lp + "self_attn_layer_norm.bias"), device),
            qkv_w=_tile(_dev(qkv_w, device), ops.TILE_ROTARY, cfg.head_dim), qkv_b=_dev(qkv_b, device),
            o_w=_tile(_dev(g(lp + "self_attn.out_proj.weight"), device)),
            o_b=_dev(g(lp + "self_attn.out_proj.bias"), device),
            mlp_norm_w=_dev(g(lp + "final_layer_norm.weight"), device),
            mlp_norm_b=_dev(g(lp + "final_layer_norm.bias"), device),
            up_w=_tile(_dev(g(lp + "fc1.weight"), device)), up_b=_dev(g(lp + "fc1.bias"), device),
            down_w=_tile(_dev(g(lp + "fc2.weight"), device)), down_b=_dev(g(lp + "fc2.bias"), device)))
    embed, lm_head, tied = _embed_and_head(_dev(g(pre + "embed_tokens.weight"), device),
                                           opt("lm_head.weight"), device, fp8, sub)
    return ModelWeights(cfg=cfg, embed=embed, embed_tiled=tied, fp8=fp8,
                        head_map=None if sub is None else sub.to(torch.int32),
                        pos_table=_dev(g(pre + "embed_positions.weight"), device),
                        final_norm_w=_dev(g(pre + "final_layer_norm.weight"), device),
                        final_norm_b=_dev(g(pre + "final_layer_norm.bias"), device),
                        lm_head=lm_head, layers=layers)


def shard_state_dict(cfg: ModelConfig, state: Dict[str, torch.Tensor], tp_size: int,
                     tp_rank: int, vocab_parallel: bool = False):
    """(per-rank config, per-rank state dict) for tensor parallelism over `tp_size` GPUs.

    Column-parallel: q/k/v projections by head and gate/up (fc1) by ffn column keep the
    rows of the rank's share; row-parallel: o_proj and down_proj (fc2) keep the matching
    input columns, their partial products are summed over the ranks.  Norms, embeddings,
    LM head and the biases of the row-parallel layers stay whole (rank 0 applies them).
    vocab_parallel: the LM head keeps only the rank's slice of vocabulary rows (a tied head
    becomes an explicit "lm_head.weight" slice; the embedding table stays whole)."""
    if not 0 <= tp_rank < tp_size:
        raise ValueError(f"tp_rank {tp_rank} outside 0..{tp_size - 1}")
    local = cfg.tp_shard(tp_size, vocab_parallel)
    D = cfg.head_dim
    q0, q1 = tp_rank * local.n_heads * D, (tp_rank + 1) * local.n_heads * D
    k0, k1 = tp_rank * local.n_kv_heads * D, (tp_rank + 1) * local.n_kv_heads * D
    f0, f1 = tp_rank * local.ffn, (tp_rank + 1) * local.ffn
    rows = {"q_proj": (q0, q1), "k_proj": (k0, k1), "v_proj": (k0, k1), "gate_proj": (f0, f1),
            "up_proj": (f0, f1), "fc1": (f0, f1)}
    cols = {"o_proj": (q0, q1), "out_proj": (q0, q1), "down_proj": (f0, f1), "fc2": (f0, f1)}
    out: Dict[str, torch.Tensor] = {}
    for name, t in state.items():
        parts = name.split(".")
        mod, kind = (parts[-2], parts[-1]) if len(parts) >= 2 else ("", "")
        if "layers" in parts and mod in rows:
            a, b = rows[mod]
            t = t[a:b]
        elif "layers" in parts and mod in cols and kind == "weight":
            a, b = cols[mod]
            t = t[:, a:b]
        out[name] = t.contiguous()
    if vocab_parallel:
        v0, v1 = tp_rank * local.lm_vocab, (tp_rank + 1) * local.lm_vocab
        head = state.get("lm_head.weight")
        if head is None:
            head = next(t for n, t in state.items() if n.endswith("embed_tokens.weight"))
        out["lm_head.weight"] = head[v0:v1].contiguous()
    return local, out


def random_init(cfg: ModelConfig, seed: int = 0, device="cuda", std: float = 0.02,
                fp8: bool = False, head_subset=None, tp_rank: int = 0) -> ModelWeights:
    """Seeded random weights generated directly on the device in the fused
    layout (no host copy: an 8B model is 16 GB).  head_subset: as for from_state_dict (the
    other tensors are those of the same seed without it).  tp_rank: cfg is one rank's share
    of a tensor-parallel model (ModelConfig.tp_shard); every rank draws the same replicated
    tensors (norms, embedding) and its own sharded matrices (rank 0's, rotated along the input
    dimension), so that the ranks' partial products differ as real shards' do."""
    cfg.validate()
    sub = None
    full_rows = cfg.head_rows
    if head_subset is not None:
        cfg, sub = _head_subset(cfg, head_subset, device)
    gen = torch.Generator(device=device).manual_seed(seed)

    def _tile(w, mode=ops.TILE_PLAIN, head_dim=0):
        return _tile_matrix(w, mode, head_dim, fp8=fp8)

    def rn(*shape, s=std, sharded=True):
        w = (torch.randn(*shape, generator=gen, device=device, dtype=torch.float32) * s
             ).to(torch.bfloat16)
        if tp_rank and sharded and len(shape) == 2:
            w = w.roll(17 * tp_rank, dims=1)
        return w

    def ones(n):
        return (1.0 + torch.randn(n, generator=gen, device=device) * 0.05).to(torch.bfloat16)

    H, F = cfg.hidden, cfg.ffn
    layers = []
    for _ in range(cfg.n_layers):
        if cfg.arch == "llama":
            layers.append(LayerTensors(
                attn_norm_w=ones(H), qkv_w=_tile(rn(cfg.qkv_rows, H), ops.TILE_ROTARY, cfg.head_dim),
                qkv_b=rn(cfg.qkv_rows) if cfg.qkv_bias else None,
                o_w=_tile(rn(H, cfg.n_heads * cfg.head_dim)), mlp_norm_w=ones(H),
                up_w=_tile(rn(2 * F, H), ops.TILE_GATED), down_w=_tile(rn(H, F))))
        else:
            layers.append(LayerTensors(
                attn_norm_w=ones(H), attn_norm_b=rn(H),
                qkv_w=_tile(rn(cfg.qkv_rows, H), ops.TILE_ROTARY, cfg.head_dim),
                qkv_b=rn(cfg.qkv_rows), o_w=_tile(rn(H, cfg.n_heads * cfg.head_dim)), o_b=rn(H),
                mlp_norm_w=ones(H), mlp_norm_b=rn(H), up_w=_tile(rn(F, H)), up_b=rn(F),
                down_w=_tile(rn(H, F)), down_b=rn(H)))
    embed = rn(cfg.vocab, H, s=1.0 if cfg.arch == "llama" else 0.5, sharded=False)
    embed, lm_head, tied = _embed_and_head(embed, None if cfg.tie_embeddings else rn(full_rows, H),
                                           device, fp8, sub)
    w = ModelWeights(cfg=cfg, embed=embed, embed_tiled=tied, final_norm_w=ones(H), lm_head=lm_head,
                     layers=layers, fp8=fp8, head_map=None if sub is None else sub.to(torch.int32))
    if cfg.arch == "llama":
        w.rope_cs = rope_table(cfg, device)
    else:
        w.pos_table = rn(cfg.max_pos + cfg.pos_bias, H, s=0.5, sharded=False)
        w.final_norm_b = rn(H)
    return w


def from_safetensors_dir(cfg: ModelConfig, model_dir: str, device="cuda",
                         fp8: bool = False, head_subset=None) -> ModelWeights:
    """Loads every *.safetensors shard of a local Hugging Face checkpoint."""
    from safetensors import safe_open

    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors under {model_dir}")
    state: Dict[str, torch.Tensor] = {}
    for fn in files:
        with safe_open(fn, framework="pt", device="cpu") as f:
            for key in f.keys():
                state[key] = f.get_tensor(key)
    if cfg.arch == "opt" and "decoder.embed_tokens.weight" in state:
        state = {"model." + k if k.startswith("decoder.") else k: v for k, v in state.items()}
    return from_state_dict(cfg, state, device, fp8=fp8, head_subset=head_subset)


# ---------------------------------------------------------------------------------------------
# Layer-list models (config.SeqModelConfig): row-major matrices in the dtype the model is served
# in (bfloat16 or float32), every matrix of a layer that reads the normed input stacked into one.
@dataclass
class SeqLayerTensors:
    norm_w: torch.Tensor
    # A matrix is either a row-major tensor or, for bfloat16 serving and an input width that is a
    # multiple of 32, an ops.TiledWeight for the MFMA linear kernels the other decoders use.
    w_in: object                  # [q | k | v | g | r1 | r2 | ff gate | ff up | a1] x width
    w_o: object
    r1_bias: torch.Tensor         # f32 [width]
    r2_bias: Optional[torch.Tensor] = None
    w_down: object = None
    w_a2: Optional[torch.Tensor] = None
    b_a2: Optional[torch.Tensor] = None       # f32
    head_decay: Optional[torch.Tensor] = None  # f32 [heads]
    head_bias: Optional[torch.Tensor] = None   # f32 [heads]
    head_norm_w: Optional[torch.Tensor] = None
    inv_freq: Optional[torch.Tensor] = None    # f64 [rot_dims / 2]
    rot_mag: float = 1.0                       # factor of cos and sin
    # layers normed on their sublayers' outputs (norm_w is norm1; r1_bias unused)
    norm2_w: Optional[torch.Tensor] = None
    dq_norm_w: Optional[torch.Tensor] = None   # latent attention
    dkv_norm_w: Optional[torch.Tensor] = None
    w_uq: object = None
    w_uk_t: Optional[torch.Tensor] = None      # [heads, kv_rank, dim]: key expansions, transposed
    w_uv: Optional[torch.Tensor] = None
    q_norm_w: Optional[torch.Tensor] = None    # attention beside a state-space recurrence
    k_norm_w: Optional[torch.Tensor] = None
    conv_w: Optional[torch.Tensor] = None
    conv_b: Optional[torch.Tensor] = None
    dt_bias: Optional[torch.Tensor] = None
    a_log: Optional[torch.Tensor] = None
    skip_d: Optional[torch.Tensor] = None
    s_norm_w: Optional[torch.Tensor] = None
    w_o2: object = None
    w_router: Optional[torch.Tensor] = None    # routed experts
    w_gate_up: Optional[torch.Tensor] = None   # [experts, 2*ff, width] ([experts, ff, width]: experts of two matrices)
    w_down_e: Optional[torch.Tensor] = None    # [experts, width, ff]
    # layers normed before and after their sublayers (norm_w / norm2_w before, these after)
    post_norm_w: Optional[torch.Tensor] = None
    post_norm2_w: Optional[torch.Tensor] = None
    sinks: Optional[torch.Tensor] = None       # f32 [heads]
    w_ff_in: object = None                     # [2*ff, width]: gate rows, then up rows
    w_shared_in: object = None                 # a shared expert: [shared_ff, width]
    w_shared_down: object = None               # [width, shared_ff]
    w_shared_gate: Optional[torch.Tensor] = None   # [1, width]
    w_in_bias: Optional[torch.Tensor] = None   # [w_in's rows]: biases of q and k
    w_o_bias: Optional[torch.Tensor] = None    # [width]
    router_bias: Optional[torch.Tensor] = None  # f32 [experts]
    diff_lambda: float = 0.0                   # differential attention: the second map's factor


@dataclass
class SeqModelWeights:
    cfg: "SeqModelConfig"
    dtype: torch.dtype
    embed: torch.Tensor
    final_norm_w: torch.Tensor
    layers: List[SeqLayerTensors]
    head_tiled: Optional["ops.TiledWeight"] = None   # the head's matrix once more, tiled
    head: Optional[torch.Tensor] = None              # an untied head, row-major
    bigram: Optional[torch.Tensor] = None            # [buckets + 1, width]
    loop_step: Optional[torch.Tensor] = None         # [times, width]: added to the stream before each pass

    def tensors(self):
        yield self.embed
        yield self.final_norm_w
        if self.head_tiled is not None:
            yield self.head_tiled.data
        for t in (self.head, self.bigram, self.loop_step):
            if t is not None:
                yield t
        for l in self.layers:
            for t in vars(l).values():
                if isinstance(t, ops.TiledWeight):
                    yield t.data
                elif isinstance(t, torch.Tensor):
                    yield t

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.tensors())


def seq_from_state_dict(cfg, state: Dict[str, torch.Tensor], device="cuda",
                        dtype: torch.dtype = torch.bfloat16, tiled: bool = True) -> SeqModelWeights:
    """Tensors under the checkpoint's names ('embed', 'final.norm', 'l<i>.norm1', 'l<i>.mix.*',
    'l<i>.mlp.*', 'l<i>.rg1', 'l<i>.rg1.b', ...) -> device tensors in the serving dtype.
    tiled=False keeps every matrix row-major (the plain kernels), whatever its shape."""
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("a layer-list model is served in bfloat16 or float32")
    W = cfg.width

    def get(name, shape):
        if name not in state:
            raise KeyError(f"checkpoint has no tensor {name!r}")
        t = state[name]
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    def dev(t, dt=None):
        return t.to(dt or dtype).contiguous().to(device)

    def mat(t):
        """A matrix [N, K] for the linear layers."""
        d = dev(t)
        if tiled and dtype == torch.bfloat16 and t.shape[1] % 32 == 0 and torch.device(device).type == "cuda":
            return ops.tile_weights(d, ops.TILE_PLAIN)
        return d

    if cfg.block == "sandwich":
        layers = [_sandwich_layer(cfg, i, get, dev, mat) for i in range(cfg.n_layers)]
        head = mat(get("head", (cfg.vocab, W)))
        return SeqModelWeights(cfg, dtype, dev(get("embed", (cfg.vocab, W))), dev(get("final.norm", (W,))), layers,
                               head if isinstance(head, ops.TiledWeight) else None, dev(get("head", (cfg.vocab, W))),
                               loop_step=dev(get("loop.step", (cfg.loop["times"], W))) if cfg.loop else None)
    if cfg.block == "postnorm":
        layers = [_postnorm_layer(cfg, i, get, dev, mat) for i in range(cfg.n_layers)]
        head_t = get("embed" if cfg.tied_head else "head", (cfg.vocab, W))
        head = mat(head_t)
        bg = cfg.bigram
        return SeqModelWeights(cfg, dtype, dev(get("embed", (cfg.vocab, W))), dev(get("final.norm", (W,))), layers,
                               head if isinstance(head, ops.TiledWeight) else None,
                               None if cfg.tied_head else dev(head_t),
                               dev(get("bigram", (bg["buckets"] + 1, W))) if bg else None)

    layers = []
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        H, G, dk, dv = m.heads, m.kv_heads, m.dim, m.vdim
        parts = [get(p + "mix.q", (H * dk, W)), get(p + "mix.k", (G * dk, W)), get(p + "mix.v", (G * dv, W)),
                 get(p + "mix.g", (H * dv, W)), get(p + "rg1", (W, W))]
        if l.ff:
            parts += [get(p + "rg2", (W, W)), get(p + "mlp.gate", (l.ff, W)), get(p + "mlp.up", (l.ff, W))]
        if m.kind == "gla":
            parts.append(get(p + "mix.a1", (m.rank, W)))
        lt = SeqLayerTensors(
            norm_w=dev(get(p + "norm1", (W,))), w_in=mat(torch.cat([t.float() for t in parts])),
            w_o=mat(get(p + "mix.o", (W, H * dv))), r1_bias=dev(get(p + "rg1.b", (W,)), torch.float32))
        if l.ff:
            lt.w_down = mat(get(p + "mlp.down", (W, l.ff)))
            lt.r2_bias = dev(get(p + "rg2.b", (W,)), torch.float32)
        if m.kind == "gla":
            lt.w_a2 = dev(get(p + "mix.a2", (H * dk, m.rank)))
            lt.b_a2 = dev(get(p + "mix.a2.b", (H * dk,)), torch.float32)
            lt.head_norm_w = dev(get(p + "mix.norm", (dv,)))
        if m.kind == "retention":
            lt.head_decay = dev(torch.tensor(m.decay, dtype=torch.float64), torch.float32)
        if m.kind == "attention":
            lt.head_bias = dev(get(p + "mix.pb", (H,)), torch.float32)
        if m.rot_dims:
            i2 = torch.arange(m.rot_dims // 2, dtype=torch.float64)
            lt.inv_freq = dev(torch.tensor(m.rot_base, dtype=torch.float64) ** (-2.0 * i2 / m.rot_dims),
                              torch.float64)
        layers.append(lt)
    embed = dev(get("embed", (cfg.vocab, W)))
    head = mat(get("embed", (cfg.vocab, W)))
    return SeqModelWeights(cfg, dtype, embed, dev(get("final.norm", (W,))), layers,
                           head if isinstance(head, ops.TiledWeight) else None)


def _postnorm_layer(cfg, i: int, get, dev, mat) -> SeqLayerTensors:
    """Layer i of a model whose layers are normed on their sublayers' outputs: the matrices that
    read the residual stacked into w_in, per-head key expansions transposed for the product
    that takes a query to the latent, the experts' matrices stacked per layer."""
    from .config import rotary_frequencies
    l, p, W = cfg.layers[i], f"l{i}.", cfg.width
    m = l.mixer
    H, dk, dv = m.heads, m.dim, m.vdim
    if m.kind == "latent_attention":
        rk, dr, qr = m.kv_rank, m.rot_dim, m.q_rank
        w_in = torch.cat([get(p + "mix.dq", (qr, W)).float(), get(p + "mix.dkv", (rk + dr, W)).float()])
        lt = SeqLayerTensors(norm_w=dev(get(p + "norm1", (W,))), w_in=mat(w_in), w_o=mat(get(p + "mix.o", (W, H * dv))),
                             r1_bias=None)
        lt.dq_norm_w, lt.dkv_norm_w = dev(get(p + "mix.dq.norm", (qr,))), dev(get(p + "mix.dkv.norm", (rk,)))
        lt.w_uq = mat(get(p + "mix.uq", (H * (dk + dr), qr)))
        lt.w_uk_t = dev(get(p + "mix.uk", (H * dk, rk)).view(H, dk, rk).transpose(1, 2))
        lt.w_uv = dev(get(p + "mix.uv", (H * dv, rk)))
        if m.rot_dims:
            f, mag = rotary_frequencies(m.rot_dims, m.rot_base, m.rot_scaling)
            lt.inv_freq, lt.rot_mag = dev(f, torch.float64), float(mag)
    else:
        G, sd = m.kv_heads, m.ssd
        w_in = torch.cat([get(p + "mix.left.q", (H * dk, W)).float(), get(p + "mix.left.k", (G * dk, W)).float(),
                          get(p + "mix.left.v", (G * dv, W)).float(),
                          get(p + "mix.right.in", (2 * sd.inner + 2 * sd.groups * sd.state + sd.heads, W)).float()])
        lt = SeqLayerTensors(norm_w=dev(get(p + "norm1", (W,))), w_in=mat(w_in),
                             w_o=mat(get(p + "mix.left.o", (W, H * dv))), r1_bias=None)
        lt.q_norm_w, lt.k_norm_w = dev(get(p + "mix.left.q.norm", (H * dk,))), dev(get(p + "mix.left.k.norm", (G * dk,)))
        lt.conv_w = dev(get(p + "mix.right.conv", (sd.conv_channels, sd.taps)))
        lt.conv_b = dev(get(p + "mix.right.conv.b", (sd.conv_channels,)))
        lt.dt_bias, lt.a_log = dev(get(p + "mix.right.dt_bias", (sd.heads,))), dev(get(p + "mix.right.A_log", (sd.heads,)))
        lt.skip_d, lt.s_norm_w = dev(get(p + "mix.right.D", (sd.heads,))), dev(get(p + "mix.right.norm", (sd.inner,)))
        lt.w_o2 = mat(get(p + "mix.right.o", (W, sd.inner)))
    ex = l.experts
    if ex is not None:
        lt.norm2_w = dev(get(p + "norm2", (W,)))
        lt.w_router = dev(get(p + "mlp.router", (ex.experts, W)))
        lt.w_gate_up = dev(torch.stack([torch.cat([get(p + f"mlp.e{e}.gate", (ex.ff, W)), get(p + f"mlp.e{e}.up", (ex.ff, W))])
                                        for e in range(ex.experts)]))
        lt.w_down_e = dev(torch.stack([get(p + f"mlp.e{e}.down", (W, ex.ff)) for e in range(ex.experts)]))
    return lt


def _sandwich_layer(cfg, i: int, get, dev, mat) -> SeqLayerTensors:
    """Layer i of a model whose layers are normed before and after their sublayers: the matrices
    that read the mixer's normed input stacked into w_in (the head gates last), per-head key
    expansions transposed, a gated feed-forward's two input matrices stacked, the experts'
    matrices stacked per layer."""
    l, p, W = cfg.layers[i], f"l{i}.", cfg.width
    m = l.mixer
    H, G, dk, dv = m.heads, m.kv_heads, m.dim, m.vdim
    if m.kind == "latent_attention":
        rk, dr = m.kv_rank, m.rot_dim
        parts = [get(p + "mix.q", (H * (dk + dr), W)), get(p + "mix.dkv", (rk + dr, W))]
        if m.head_gate:
            parts.append(get(p + "mix.g", (H, W)))
        lt = SeqLayerTensors(norm_w=dev(get(p + "norm1", (W,))), w_in=mat(torch.cat([t.float() for t in parts])),
                             w_o=mat(get(p + "mix.o", (W, H * dv))), r1_bias=None)
        lt.dkv_norm_w = dev(get(p + "mix.dkv.norm", (rk,)))
        lt.w_uk_t = dev(get(p + "mix.uk", (H * dk, rk)).view(H, dk, rk).transpose(1, 2))
        lt.w_uv = dev(get(p + "mix.uv", (H * dv, rk)))
        if m.sink:
            lt.sinks = dev(get(p + "mix.sink", (H,)), torch.float32)
        if m.rot_dims:
            i2 = torch.arange(m.rot_dims // 2, dtype=torch.float64)
            lt.inv_freq = dev(torch.tensor(m.rot_base, dtype=torch.float64) ** (-2.0 * i2 / m.rot_dims), torch.float64)
    else:
        from .config import rotary_frequencies
        own, nq, nk = m.kv_from < 0, H * m.maps * dk, G * m.maps * dk
        parts = [get(p + "mix.q", (nq, W))]
        if own:
            parts += [get(p + "mix.k", (nk, W))] + ([] if m.value_is_key else [get(p + "mix.v", (G * dv, W))])
        lt = SeqLayerTensors(norm_w=dev(get(p + "norm1", (W,))), w_in=mat(torch.cat([t.float() for t in parts])),
                             w_o=mat(get(p + "mix.o", (W, H * dv))), r1_bias=None)
        if m.qk_head_norm or m.qk_full_norm:
            n1, n2 = (dk, dk) if m.qk_head_norm else (nq, nk)
            lt.q_norm_w = dev(get(p + "mix.q.norm", (n1,)))
            lt.k_norm_w = dev(get(p + "mix.k.norm", (n2,))) if own else None
        if m.proj_bias:
            rows = [get(p + "mix.q.b", (nq,))] + ([get(p + "mix.k.b", (nk,))] if own else [])
            if own and not m.value_is_key:
                rows.append(torch.zeros(G * dv))
            lt.w_in_bias = dev(torch.cat([t.float() for t in rows]))
            lt.w_o_bias = dev(get(p + "mix.o.b", (W,)))
        if m.unit_sink:
            lt.sinks = dev(torch.zeros(H * m.maps), torch.float32)
        if m.maps == 2:
            # one number per layer, formed in float32 from the four learned vectors
            lq1, lk1, lq2, lk2 = (get(p + "mix." + n, (dk,)).float() for n in ("lq1", "lk1", "lq2", "lk2"))
            lt.diff_lambda = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + torch.tensor(m.diff))
        if m.rot_dims:
            f, mag = rotary_frequencies(m.rot_dims, m.rot_base, m.rot_scaling)
            lt.inv_freq, lt.rot_mag = dev(f, torch.float64), float(mag)
    lt.post_norm_w = dev(get(p + "norm1b", (W,)))
    ex = l.experts
    if l.ff or ex is not None:
        lt.norm2_w, lt.post_norm2_w = dev(get(p + "norm2", (W,))), dev(get(p + "norm2b", (W,)))
    if l.ff:
        lt.w_ff_in = mat(torch.cat([get(p + "mlp.gate", (l.ff, W)).float(), get(p + "mlp.up", (l.ff, W)).float()]))
        lt.w_down = mat(get(p + "mlp.down", (W, l.ff)))
    if ex is not None:
        gated = ex.act == "silu"
        lt.w_router = dev(get(p + "mlp.router", (ex.experts, W)))
        if ex.router_bias:
            lt.router_bias = dev(get(p + "mlp.router.b", (ex.experts,)), torch.float32)
        lt.w_gate_up = dev(torch.stack([
            torch.cat([get(p + f"mlp.e{e}.gate", (ex.ff, W)), get(p + f"mlp.e{e}.up", (ex.ff, W))]) if gated
            else get(p + f"mlp.e{e}.up", (ex.ff, W)) for e in range(ex.experts)]))
        lt.w_down_e = dev(torch.stack([get(p + f"mlp.e{e}.down", (W, ex.ff)) for e in range(ex.experts)]))
        if ex.shared_ff:
            F = ex.shared_ff
            lt.w_shared_in = mat(torch.cat([get(p + "mlp.shared.gate", (F, W)).float(), get(p + "mlp.shared.up", (F, W)).float()])
                                 if gated else get(p + "mlp.shared.up", (F, W)))
            lt.w_shared_down = mat(get(p + "mlp.shared.down", (W, F)))
            if ex.shared_gate:
                lt.w_shared_gate = dev(get(p + "mlp.shared.sg", (1, W)))
    return lt


def seq_from_safetensors_dir(cfg, model_dir: str, device="cuda",
                             dtype: torch.dtype = torch.bfloat16) -> SeqModelWeights:
    from safetensors import safe_open

    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no *.safetensors under {model_dir}")
    state: Dict[str, torch.Tensor] = {}
    for fn in files:
        with safe_open(fn, framework="pt", device="cpu") as f:
            for key in f.keys():
                state[key] = f.get_tensor(key)
    return seq_from_state_dict(cfg, state, device, dtype)


def seq_random_state(cfg, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Seeded random tensors under the checkpoint's names (bfloat16 values), scaled so that
    activations stay of order one: for benchmarks and examples."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def rn(*shape, s):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    if cfg.block == "postnorm":
        return _postnorm_random_state(cfg, rn)
    if cfg.block == "sandwich":
        return _sandwich_random_state(cfg, rn)
    st = {"embed": rn(cfg.vocab, W, s=1.0), "final.norm": rn(W, s=0.1)}
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        H, G, dk, dv = m.heads, m.kv_heads, m.dim, m.vdim
        st[p + "norm1"] = rn(W, s=0.1)
        for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv), ("g", H * dv)):
            st[p + "mix." + nm] = rn(rows, W, s=W ** -0.5)
        st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        if m.kind == "attention":
            st[p + "mix.pb"] = rn(H, s=1.0) - 4.0
        if m.kind == "gla":
            st[p + "mix.norm"] = 1 + rn(dv, s=0.1)
            st[p + "mix.a1"] = rn(m.rank, W, s=W ** -0.5)
            st[p + "mix.a2"] = rn(H * dk, m.rank, s=m.rank ** -0.5)
            st[p + "mix.a2.b"] = rn(H * dk, s=1.0) + 3.0
        st[p + "rg1"], st[p + "rg1.b"] = rn(W, W, s=W ** -0.5), rn(W, s=0.5)
        if l.ff:
            st[p + "mlp.gate"], st[p + "mlp.up"] = rn(l.ff, W, s=W ** -0.5), rn(l.ff, W, s=W ** -0.5)
            st[p + "mlp.down"] = rn(W, l.ff, s=l.ff ** -0.5)
            st[p + "rg2"], st[p + "rg2.b"] = rn(W, W, s=W ** -0.5), rn(W, s=0.5)
    return st


def _postnorm_random_state(cfg, rn) -> Dict[str, torch.Tensor]:
    W = cfg.width
    st = {"embed": rn(cfg.vocab, W, s=1.0), "final.norm": 1 + rn(W, s=0.1)}
    if not cfg.tied_head:
        st["head"] = rn(cfg.vocab, W, s=W ** -0.5)
    if cfg.bigram:
        st["bigram"] = rn(cfg.bigram["buckets"] + 1, W, s=0.5)
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        H, dk, dv = m.heads, m.dim, m.vdim
        st[p + "norm1"] = 1 + rn(W, s=0.1)
        if m.kind == "latent_attention":
            rk, dr, qr = m.kv_rank, m.rot_dim, m.q_rank
            st[p + "mix.dq"], st[p + "mix.dq.norm"] = rn(qr, W, s=W ** -0.5), 1 + rn(qr, s=0.1)
            st[p + "mix.uq"] = rn(H * (dk + dr), qr, s=qr ** -0.5)
            st[p + "mix.dkv"], st[p + "mix.dkv.norm"] = rn(rk + dr, W, s=W ** -0.5), 1 + rn(rk, s=0.1)
            st[p + "mix.uk"], st[p + "mix.uv"] = rn(H * dk, rk, s=rk ** -0.5), rn(H * dv, rk, s=rk ** -0.5)
            st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        else:
            G, sd = m.kv_heads, m.ssd
            st[p + "mix.left.q"], st[p + "mix.left.k"] = rn(H * dk, W, s=W ** -0.5), rn(G * dk, W, s=W ** -0.5)
            st[p + "mix.left.v"] = rn(G * dv, W, s=W ** -0.5)
            st[p + "mix.left.q.norm"], st[p + "mix.left.k.norm"] = 1 + rn(H * dk, s=0.1), 1 + rn(G * dk, s=0.1)
            st[p + "mix.left.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
            st[p + "mix.right.in"] = rn(2 * sd.inner + 2 * sd.groups * sd.state + sd.heads, W, s=W ** -0.5)
            st[p + "mix.right.conv"], st[p + "mix.right.conv.b"] = rn(sd.conv_channels, sd.taps, s=0.5), rn(sd.conv_channels, s=0.1)
            st[p + "mix.right.dt_bias"], st[p + "mix.right.A_log"] = rn(sd.heads, s=0.5) - 1.0, rn(sd.heads, s=0.5) - 1.0
            st[p + "mix.right.D"], st[p + "mix.right.norm"] = 1 + rn(sd.heads, s=0.2), 1 + rn(sd.inner, s=0.1)
            st[p + "mix.right.o"] = rn(W, sd.inner, s=sd.inner ** -0.5)
        ex = l.experts
        if ex is not None:
            st[p + "norm2"], st[p + "mlp.router"] = 1 + rn(W, s=0.1), rn(ex.experts, W, s=W ** -0.5)
            for e in range(ex.experts):
                st[p + f"mlp.e{e}.gate"], st[p + f"mlp.e{e}.up"] = rn(ex.ff, W, s=W ** -0.5), rn(ex.ff, W, s=W ** -0.5)
                st[p + f"mlp.e{e}.down"] = rn(W, ex.ff, s=ex.ff ** -0.5)
    return st


def _sandwich_random_state(cfg, rn) -> Dict[str, torch.Tensor]:
    W = cfg.width
    st = {"embed": rn(cfg.vocab, W, s=1.0), "final.norm": 1 + rn(W, s=0.1), "head": rn(cfg.vocab, W, s=W ** -0.5)}
    if cfg.loop:
        st["loop.step"] = rn(cfg.loop["times"], W, s=0.5)
    for i, l in enumerate(cfg.layers):
        m, p = l.mixer, f"l{i}."
        H, G, dk, dv = m.heads, m.kv_heads, m.dim, m.vdim
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if (l.ff or l.experts) else ()):
            st[p + nm] = 1 + rn(W, s=0.1)
        if m.kind == "latent_attention":
            rk, dr = m.kv_rank, m.rot_dim
            st[p + "mix.q"] = rn(H * (dk + dr), W, s=W ** -0.5)
            st[p + "mix.dkv"], st[p + "mix.dkv.norm"] = rn(rk + dr, W, s=W ** -0.5), 1 + rn(rk, s=0.1)
            st[p + "mix.uk"], st[p + "mix.uv"] = rn(H * dk, rk, s=rk ** -0.5), rn(H * dv, rk, s=rk ** -0.5)
            if m.sink:
                st[p + "mix.sink"] = rn(H, s=1.0)
            if m.head_gate:
                st[p + "mix.g"] = rn(H, W, s=W ** -0.5)
        else:
            own, nq, nk = m.kv_from < 0, H * m.maps * dk, G * m.maps * dk
            st[p + "mix.q"] = rn(nq, W, s=W ** -0.5)
            if own:
                st[p + "mix.k"] = rn(nk, W, s=W ** -0.5)
                if not m.value_is_key:
                    st[p + "mix.v"] = rn(G * dv, W, s=W ** -0.5)
            if m.qk_head_norm or m.qk_full_norm:
                st[p + "mix.q.norm"] = 1 + rn(dk if m.qk_head_norm else nq, s=0.1)
                if own:
                    st[p + "mix.k.norm"] = 1 + rn(dk if m.qk_head_norm else nk, s=0.1)
            if m.proj_bias:
                st[p + "mix.q.b"], st[p + "mix.o.b"] = rn(nq, s=0.2), rn(W, s=0.2)
                if own:
                    st[p + "mix.k.b"] = rn(nk, s=0.2)
            if m.maps == 2:
                for nm in ("lq1", "lk1", "lq2", "lk2"):
                    st[p + "mix." + nm] = rn(dk, s=0.3)
        st[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        if l.ff:
            st[p + "mlp.gate"], st[p + "mlp.up"] = rn(l.ff, W, s=W ** -0.5), rn(l.ff, W, s=W ** -0.5)
            st[p + "mlp.down"] = rn(W, l.ff, s=l.ff ** -0.5)
        ex = l.experts
        if ex is not None:
            st[p + "mlp.router"] = rn(ex.experts, W, s=W ** -0.5)
            if ex.router_bias:
                st[p + "mlp.router.b"] = rn(ex.experts, s=0.3)
            names = [f"e{e}" for e in range(ex.experts)] + (["shared"] if ex.shared_ff else [])
            for nm in names:
                F = ex.shared_ff if nm == "shared" else ex.ff
                if ex.act == "silu":
                    st[p + f"mlp.{nm}.gate"] = rn(F, W, s=W ** -0.5)
                st[p + f"mlp.{nm}.up"], st[p + f"mlp.{nm}.down"] = rn(F, W, s=W ** -0.5), rn(W, F, s=F ** -0.5)
            if ex.shared_ff and ex.shared_gate:
                st[p + "mlp.shared.sg"] = rn(1, W, s=W ** -0.5)
    return st


def load_model(model_dir: str, device="cuda", dtype: torch.dtype = torch.bfloat16, **kw):
    """Configuration and weights of a checkpoint folder, whatever model class its config.json
    names: (SeqModelConfig, SeqModelWeights) or (ModelConfig, ModelWeights)."""
    from .config import SeqModelConfig, load_model_config
    cfg = load_model_config(model_dir)
    if isinstance(cfg, SeqModelConfig):
        return cfg, seq_from_safetensors_dir(cfg, model_dir, device, dtype)
    if dtype != torch.bfloat16:
        raise ValueError("Hugging Face decoders are served in bfloat16 (or fp8 weights) only")
    return cfg, from_safetensors_dir(cfg, model_dir, device, **kw)
