"""Model and engine configuration.

Configuration style mirrors the reference's: a dataclass with keyword
overrides and a ValueError on unknown keys
(/root/reference/src/qwen_image_gen/config.py:34-66).
"""
from __future__ import annotations

import json
import math
import os
import dataclasses
from dataclasses import dataclass, field, fields
from typing import List, Optional

import torch


@dataclass
class ModelConfig:
    arch: str = "llama"            # "llama" (Llama, Qwen2) or "opt"
    n_layers: int = 2
    hidden: int = 128
    n_heads: int = 2
    n_kv_heads: int = 2
    head_dim: int = 64
    ffn: int = 256
    vocab: int = 256
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[dict] = None
    max_pos: int = 2048
    tie_embeddings: bool = False
    qkv_bias: bool = False
    pos_bias: int = 2              # OPT learned-position offset
    name: str = "custom"
    # Vocabulary-parallel LM head (tensor parallelism): rows of the head one rank holds;
    # 0 = the whole vocabulary.  The embedding table is never split.
    lm_vocab: int = 0
    # Multimodal rotary embedding (Qwen2-VL): frequency counts of the temporal, height and
    # width position components, summing to head_dim / 2; None = ordinary rotary embedding.
    mrope_section: Optional[tuple] = None

    def validate(self) -> None:
        if self.arch not in ("llama", "opt"):
            raise ValueError(f"unknown arch {self.arch!r}")
        if self.head_dim not in (64, 128):
            raise ValueError(f"head_dim {self.head_dim} not supported (64 or 128)")
        if self.n_heads % self.n_kv_heads:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        if self.hidden % 32 or self.ffn % 32 or self.vocab % 16:
            raise ValueError("hidden and ffn must be multiples of 32, vocab a multiple of 16")
        if self.mrope_section is not None:
            sec = tuple(int(v) for v in self.mrope_section)
            if self.arch != "llama" or len(sec) != 3 or min(sec) < 0 or sum(sec) != self.head_dim // 2:
                raise ValueError(f"mrope_section {self.mrope_section} must be three counts summing "
                                 f"to head_dim/2 = {self.head_dim // 2} on a rotary model")
            self.mrope_section = sec

    @property
    def qkv_rows(self) -> int:
        return (self.n_heads + 2 * self.n_kv_heads) * self.head_dim

    def param_bytes(self) -> int:
        """bf16 bytes one forward pass streams (each matrix once; a tied head
        is read twice: as embedding rows it is negligible, as LM head in full)."""
        H, F, V = self.hidden, self.ffn, self.vocab
        per_layer = self.qkv_rows * H + H * self.n_heads * self.head_dim
        per_layer += (3 if self.arch == "llama" else 2) * F * H
        return 2 * (self.n_layers * per_layer + V * H)

    def kv_bytes_per_token(self) -> int:
        return 2 * self.n_layers * self.n_kv_heads * self.head_dim * 2

    @property
    def head_rows(self) -> int:
        """Rows of the LM head (= columns of the logits) this model instance computes."""
        return self.lm_vocab or self.vocab

    def tp_shard(self, tp_size: int, vocab_parallel: bool = False) -> "ModelConfig":
        """The per-rank view under tensor parallelism: heads and ffn columns divided,
        hidden size, vocabulary and layer count unchanged; with vocab_parallel the LM head
        is cut into tp_size row slices (each a multiple of 16 rows)."""
        if vocab_parallel and self.vocab % (16 * tp_size):
            raise ValueError(f"vocab {self.vocab} must be a multiple of 16 * tp_size for a "
                             "vocabulary-parallel head")
        if tp_size < 1 or self.n_heads % tp_size or self.n_kv_heads % tp_size:
            raise ValueError(f"tp_size {tp_size} must divide n_heads={self.n_heads} and "
                             f"n_kv_heads={self.n_kv_heads}")
        if self.ffn % (32 * tp_size):
            raise ValueError(f"ffn {self.ffn} must be a multiple of 32 * tp_size")
        return dataclasses.replace(self, n_heads=self.n_heads // tp_size,
                                   n_kv_heads=self.n_kv_heads // tp_size,
                                   ffn=self.ffn // tp_size, name=f"{self.name}/tp{tp_size}",
                                   lm_vocab=self.vocab // tp_size if vocab_parallel else 0)


def create_model_config(base: Optional[ModelConfig] = None, **overrides) -> ModelConfig:
    cfg = ModelConfig(**{f.name: getattr(base, f.name) for f in fields(ModelConfig)}) \
        if base is not None else ModelConfig()
    valid = {f.name for f in fields(ModelConfig)}
    for k, v in overrides.items():
        if k not in valid:
            raise ValueError(f"Unknown config parameter: {k}")
        setattr(cfg, k, v)
    cfg.validate()
    return cfg


_LLAMA3_SCALING = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

# Shapes of the public Hugging Face configs of the models the benchmark names.
PRESETS = {
    "llama-3-8b": dict(arch="llama", n_layers=32, hidden=4096, n_heads=32, n_kv_heads=8,
                       head_dim=128, ffn=14336, vocab=128256, rope_theta=500000.0,
                       norm_eps=1e-5, max_pos=8192),
    "llama-3.2-1b": dict(arch="llama", n_layers=16, hidden=2048, n_heads=32, n_kv_heads=8,
                         head_dim=64, ffn=8192, vocab=128256, rope_theta=500000.0,
                         rope_scaling=_LLAMA3_SCALING, norm_eps=1e-5, tie_embeddings=True,
                         max_pos=8192),
    "llama-3-70b": dict(arch="llama", n_layers=80, hidden=8192, n_heads=64, n_kv_heads=8,
                        head_dim=128, ffn=28672, vocab=128256, rope_theta=500000.0,
                        norm_eps=1e-5, max_pos=8192),
    "qwen2.5-7b": dict(arch="llama", n_layers=28, hidden=3584, n_heads=28, n_kv_heads=4,
                       head_dim=128, ffn=18944, vocab=152064, rope_theta=1000000.0,
                       norm_eps=1e-6, qkv_bias=True, max_pos=8192),
    "qwen2.5-0.5b": dict(arch="llama", n_layers=24, hidden=896, n_heads=14, n_kv_heads=2,
                         head_dim=64, ffn=4864, vocab=151936, rope_theta=1000000.0,
                         norm_eps=1e-6, qkv_bias=True, tie_embeddings=True, max_pos=8192),
    # the language model of Qwen2-VL-7B (vision tower: vision.VisionConfig)
    "qwen2-vl-7b": dict(arch="llama", n_layers=28, hidden=3584, n_heads=28, n_kv_heads=4,
                        head_dim=128, ffn=18944, vocab=152064, rope_theta=1000000.0,
                        norm_eps=1e-6, qkv_bias=True, max_pos=8192, mrope_section=(16, 24, 24)),
    "opt-125m": dict(arch="opt", n_layers=12, hidden=768, n_heads=12, n_kv_heads=12,
                     head_dim=64, ffn=3072, vocab=50272, norm_eps=1e-5, tie_embeddings=True,
                     max_pos=2048),
}


def preset(name: str, **overrides) -> ModelConfig:
    if name not in PRESETS:
        raise ValueError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    return create_model_config(None, name=name, **{**PRESETS[name], **overrides})


def from_hf_config(cfg: dict, **overrides) -> ModelConfig:
    """Builds a ModelConfig from a Hugging Face config.json dict."""
    mt = cfg.get("model_type", "llama")
    if mt == "opt":
        kw = dict(arch="opt", n_layers=cfg["num_hidden_layers"], hidden=cfg["hidden_size"],
                  n_heads=cfg["num_attention_heads"], n_kv_heads=cfg["num_attention_heads"],
                  head_dim=cfg["hidden_size"] // cfg["num_attention_heads"], ffn=cfg["ffn_dim"],
                  vocab=cfg["vocab_size"], max_pos=cfg["max_position_embeddings"],
                  tie_embeddings=cfg.get("tie_word_embeddings", True), norm_eps=1e-5)
        if cfg.get("word_embed_proj_dim", cfg["hidden_size"]) != cfg["hidden_size"]:
            raise ValueError("OPT variants with word_embed_proj_dim != hidden_size are not supported")
        if not cfg.get("do_layer_norm_before", True):
            raise ValueError("post-LN OPT variants are not supported")
    elif mt in ("llama", "qwen2", "mistral", "qwen2_vl", "qwen2_5_vl", "qwen2_vl_text",
                "qwen2_5_vl_text"):
        vl = mt.startswith("qwen2_")
        if vl and "text_config" in cfg:   # newer checkpoints nest the language model's fields
            cfg = {**cfg, **cfg["text_config"]}
        nh = cfg["num_attention_heads"]
        kw = dict(arch="llama", n_layers=cfg["num_hidden_layers"], hidden=cfg["hidden_size"],
                  n_heads=nh, n_kv_heads=cfg.get("num_key_value_heads", nh),
                  head_dim=cfg.get("head_dim") or cfg["hidden_size"] // nh,
                  ffn=cfg["intermediate_size"], vocab=cfg["vocab_size"],
                  norm_eps=cfg.get("rms_norm_eps", 1e-5), rope_theta=cfg.get("rope_theta", 10000.0),
                  rope_scaling=cfg.get("rope_scaling"),
                  max_pos=min(cfg.get("max_position_embeddings", 8192), 32768),
                  tie_embeddings=cfg.get("tie_word_embeddings", False),
                  qkv_bias=(mt == "qwen2") or vl or bool(cfg.get("attention_bias", False)))
        sc = cfg.get("rope_scaling") or {}
        if sc.get("mrope_section"):
            kw["mrope_section"] = tuple(sc["mrope_section"])
    else:
        raise ValueError(f"unsupported model_type {mt!r}")
    kw.update(overrides)
    return create_model_config(None, name=cfg.get("_name_or_path", mt), **kw)


def load_hf_config(model_dir: str, **overrides) -> ModelConfig:
    with open(os.path.join(model_dir, "config.json")) as f:
        return from_hf_config(json.load(f), **overrides)


def rope_table(cfg: ModelConfig, device="cpu") -> torch.Tensor:
    """[max_pos, head_dim] float32: cos of the D/2 rotary angles, then sin.
    Handles the "llama3" frequency rescaling of Llama-3.1/3.2 configs."""
    d = cfg.head_dim
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    sc = cfg.rope_scaling
    if sc:
        kind = sc.get("rope_type", sc.get("type"))
        if kind == "llama3":
            old = sc["original_max_position_embeddings"]
            lo_w, hi_w = old / sc["low_freq_factor"], old / sc["high_freq_factor"]
            wl = 2 * math.pi / inv
            smooth = (old / wl - sc["low_freq_factor"]) / (sc["high_freq_factor"] - sc["low_freq_factor"])
            scaled = torch.where(wl > lo_w, inv / sc["factor"], inv)
            blend = (1 - smooth) * inv / sc["factor"] + smooth * inv
            inv = torch.where((wl <= lo_w) & (wl >= hi_w), blend, scaled)
        elif kind not in (None, "default", "mrope"):  # mrope: plain frequencies, 3 positions
            raise ValueError(f"rope scaling {kind!r} not supported")
    ang = torch.arange(cfg.max_pos, dtype=torch.float32)[:, None] * inv.float()[None, :]
    return torch.cat([ang.cos(), ang.sin()], dim=1).contiguous().to(device)


# ---------------------------------------------------------------------------------------------
# Decoders described layer by layer (recurrent and windowed mixers); served by seq_engine.SeqEngine.
MIXER_KINDS = ("retention", "gla", "attention", "latent_attention", "parallel", "softmax_attention")


@dataclass
class SsdSpec:
    """A state-space recurrence with a scalar decay per head (the state-space-duality form):
    S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x; x, B, C pass a causal convolution of
    `taps` taps and silu; the output is gated by silu(z) and RMS-normed in `norm_groups` parts."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    taps: int = 4
    norm_groups: int = 1

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    def validate(self) -> None:
        if min(self.heads, self.vdim, self.state, self.groups, self.taps, self.norm_groups) < 1:
            raise ValueError("state-space sizes must be positive")
        if self.heads % self.groups or self.inner % self.norm_groups:
            raise ValueError("state-space heads must divide into groups, and the inner size into norm groups")
        if self.state > 256:
            raise ValueError("a state size above 256 is not supported")


@dataclass
class ExpertsSpec:
    """Routed experts as a layer's feed-forward: `top` of `experts` gated feed-forwards of width
    `ff` per token.  score: "sigmoid" or "softmax" over the router's logits; renorm: the chosen
    weights are divided by their sum; scale_input: the weight multiplies the expert's input
    (else its output).  act "silu": an expert is down(silu(gate h) * (up h)); "relu2": an expert has
    two matrices, down(relu(up h)^2).  The chosen weights are divided by (their sum + renorm_eps)
    when renorm, then multiplied by scale.  shared_ff > 0: one more expert of that width and the
    same form runs for every token and is added, times sigmoid(g . h) when shared_gate.  A softmax
    score that is renormed over the chosen experts is the softmax over the chosen logits alone."""
    experts: int
    top: int
    ff: int
    score: str = "sigmoid"
    renorm: bool = False
    scale_input: bool = True
    act: str = "silu"
    renorm_eps: float = 0.0
    scale: float = 1.0
    shared_ff: int = 0
    shared_gate: bool = True
    router_bias: bool = False      # a bias on the router's logits

    def validate(self) -> None:
        if self.experts < 1 or not 1 <= self.top <= self.experts or self.ff < 1 or self.shared_ff < 0:
            raise ValueError(f"experts {self.experts}, top {self.top}, ff {self.ff}, shared ff {self.shared_ff}")
        if self.score not in ("sigmoid", "softmax"):
            raise ValueError(f"unknown router score {self.score!r}")
        if self.act not in ("silu", "relu2"):
            raise ValueError(f"unknown expert activation {self.act!r}")


@dataclass
class MixerSpec:
    """One layer's token mixer.  kind "retention": decayed linear attention with a fixed decay per
    head and rotate-half rotary positions; "gla": decayed linear attention whose decay per key
    channel comes from the input through a low-rank pair of matrices (sigmoid(z)^(1/tau));
    "attention": grouped-query attention over a sliding window plus mean-pooled blocks of the
    tokens before it, with sigmoid weights, interleaved rotary positions and unit-norm q / k;
    "latent_attention": softmax attention over a sliding window whose keys and values are
    expanded from one cached latent of kv_rank channels per token, plus rot_dim rotated channels
    shared by the heads (queries through a latent of q_rank channels; dim counts the unrotated
    channels of a head); "parallel": grouped-query softmax attention without rotation, q and k
    normed over the whole projection, over a window that also keeps the first keep_first tokens,
    beside a state-space recurrence (ssd) on the same input, summed with two scales;
    "softmax_attention": grouped-query softmax attention without rotation, q and k normed per
    head with one weight of `dim` channels each (qk_head_norm), scores capped by softcap *
    tanh(s / softcap), keys of the query's own chunk of `chunk` positions only.  A latent
    attention with q_rank 0 projects its queries straight from the input; window 0 sees every
    earlier token; sink: a learned term per head in the softmax's denominator; head_gate: a
    head's output is multiplied by the sigmoid of a product of the input.  A softmax attention
    may also: rotate the leading rot_dims channels of q and k (rot_layout, rot_base, rot_scaling);
    hold `maps` score maps per head over the same values (2: differential attention, map 0's output
    minus lambda times map 1's, the difference divided by its root mean square and multiplied by
    1 - diff; lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff from four learned vectors); norm q and
    k over the whole projection (qk_full_norm); add biases to the q, k and output projections
    (proj_bias); take its values from the keys as projected (value_is_key: no value matrix); keep
    one term of score 0 in the softmax's denominator (unit_sink); read the keys and values that
    layer kv_from cached instead of projecting its own."""
    kind: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0              # 0: as many as heads
    rot_dims: int = 0              # leading channels of a head that are rotated (0: none)
    rot_base: float = 10000.0
    rot_layout: str = "half"       # "half": channel i pairs with i + rot_dims/2; "interleaved": 2i with 2i+1
    decay: Optional[tuple] = None  # retention: one factor per head
    tau: float = 1.0               # gla
    rank: int = 0                  # gla: inner size of the low-rank pair (a tensor's shape gives it)
    scale: float = 1.0             # attention: factor of the scores
    window: int = 0                # attention: tokens seen, the current one included
    pool: int = 1                  # attention: tokens per pooled block
    keep_first: int = 0            # parallel: the first tokens stay visible behind the window
    q_rank: int = 0                # latent_attention
    kv_rank: int = 0
    rot_dim: int = 0               # latent_attention: rotated channels per head (behind the `dim` unrotated)
    rot_scaling: Optional[dict] = None  # frequency blending {factor, original, fast, slow}
    ssd: Optional[SsdSpec] = None  # parallel
    left_scale: float = 1.0        # parallel: factor of the attention
    right_scale: float = 1.0       # parallel: factor of the recurrence
    chunk: int = 0                 # softmax attention: keys of the query's own chunk only (0: no chunks)
    softcap: float = 0.0           # scores capped by softcap * tanh(s / softcap) (0: not capped)
    sink: bool = False             # a learned term per head in the softmax's denominator
    head_gate: bool = False        # outputs gated per head
    qk_head_norm: bool = False     # q and k normed per head
    maps: int = 1                  # softmax attention: score maps per head
    diff: float = 0.0              # differential attention's constant
    qk_full_norm: bool = False     # q and k normed over the whole projection
    proj_bias: bool = False        # biases on the q, k and output projections
    value_is_key: bool = False     # values are the keys as projected
    unit_sink: bool = False        # one term exp(0) in the softmax's denominator
    kv_from: int = -1              # the layer whose cached keys and values this one reads (-1: its own)

    def validate(self) -> None:
        if self.kind not in MIXER_KINDS:
            raise ValueError(f"unknown mixer {self.kind!r}; known: {MIXER_KINDS}")
        self.kv_heads = self.kv_heads or self.heads
        if min(self.heads, self.kv_heads, self.dim, self.vdim) < 1 or self.heads % self.kv_heads:
            raise ValueError(f"mixer sizes: heads {self.heads}, kv_heads {self.kv_heads}, dim {self.dim}, "
                             f"vdim {self.vdim}")
        if self.rot_layout not in ("half", "interleaved"):
            raise ValueError(f"unknown rotary layout {self.rot_layout!r}")
        if self.kind == "latent_attention":
            if self.q_rank < 0 or self.kv_rank < 1 or self.rot_dim < 0 or self.window < 0:
                raise ValueError("latent attention needs q_rank >= 0, kv_rank >= 1, rot_dim >= 0, window >= 0")
            if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.rot_dim:
                raise ValueError(f"rot_dims {self.rot_dims} must be even and at most rot_dim {self.rot_dim}")
            if self.kv_rank > 512 or self.kv_heads != self.heads:
                raise ValueError("latent attention: kv_rank above 512, or kv_heads given")
            return
        if self.kind == "softmax_attention":
            if self.window < 0 or self.chunk < 0 or self.softcap < 0 or self.vdim > 512:
                raise ValueError("softmax attention needs window >= 0, chunk >= 0, softcap >= 0, vdim <= 512")
            if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
                raise ValueError(f"rot_dims {self.rot_dims} must be even and at most dim {self.dim}")
            if self.maps not in (1, 2) or (self.qk_head_norm and self.qk_full_norm) or (self.sink and self.unit_sink):
                raise ValueError("softmax attention: one or two score maps, one kind of q/k norm, one kind of sink")
            if self.value_is_key and (self.maps != 1 or self.vdim != self.dim or self.kv_from >= 0):
                raise ValueError("values taken from the keys need one score map, vdim == dim and keys of the layer's own")
            return
        if self.kind == "parallel":
            if self.window < 1 or self.keep_first < 0 or self.rot_dims or self.ssd is None or self.vdim > 512:
                raise ValueError("a parallel mixer needs window >= 1, keep_first >= 0, no rotation, vdim <= 512 "
                                 "and a state-space part")
            self.ssd.validate()
            return
        if self.rot_dims < 0 or self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ValueError(f"rot_dims {self.rot_dims} must be even and at most dim {self.dim}")
        if self.kind == "attention":
            if self.window < 1 or self.pool < 1:
                raise ValueError("an attention mixer needs window >= 1 and pool >= 1")
            if self.vdim > 256:
                raise ValueError("attention vdim above 256 is not supported")
        else:
            if self.kv_heads != self.heads:
                raise ValueError("a recurrent mixer has one key head per query head")
            if self.dim > 256:
                raise ValueError("recurrent key size above 256 is not supported")
        if self.kind == "retention":
            if self.decay is None or len(self.decay) != self.heads:
                raise ValueError("retention needs one decay per head")
            self.decay = tuple(float(d) for d in self.decay)
        if self.kind == "gla" and not self.tau > 0:
            raise ValueError("gla needs tau > 0")


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict] = None):
    """(frequencies of the dims/2 pairs as float64, factor of cos and sin).  Plain: base^(-2i/dims)
    and 1.  With scaling {factor, original, fast, slow}: pair i keeps its frequency f_i where it
    turns fast and takes f_i / factor where it turns slowly, blended along a ramp over the pair
    index between the pairs that make `fast` and `slow` turns over `original` positions; cos and
    sin grow by 0.1 ln(factor) + 1.  With scaling {factor} alone every frequency is f_i / factor."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    if "original" not in scaling:
        return f / float(scaling["factor"]), 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_index(turns: float) -> float:
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


@dataclass
class SeqLayerSpec:
    mixer: MixerSpec
    ff: int = 0                    # width of the gated feed-forward beside the mixer; 0: none
    experts: Optional[ExpertsSpec] = None   # routed experts as the feed-forward
    ff_act: str = "relu"           # the gated feed-forward's activation: "relu" or "silu"


@dataclass
class SeqModelConfig:
    """A decoder as a list of layers.  Every layer is  h = norm(x);  x += sigmoid(R1 h + r1) *
    mixer(h) + sigmoid(R2 h + r2) * ff(h)  with an RMS norm whose weight is stored around zero;
    the output head is the embedding table."""
    arch: str
    width: int
    vocab: int
    layers: List["SeqLayerSpec"]
    norm_eps: float = 1e-5
    name: str = "custom"
    # "gated": the layer above.  "postnorm": x += norm1(mixer(x)); x += norm2(ff(x)), plain norm
    # weights, the sublayers read x itself; the feed-forward is a set of routed experts or absent.
    # "sandwich": x += norm1b(mixer(norm1(x))); x += norm2b(ff(norm2(x))), plain norm weights; the
    # feed-forward is gated, a set of routed experts (with or without a shared one), or absent.
    block: str = "gated"
    embed_scale: float = 1.0
    bigram: Optional[dict] = None  # {buckets, mul_prev, mul_cur}: a hashed table of token pairs added to the embedding
    tied_head: bool = True         # False: the output head is its own tensor
    logit_scale: float = 1.0
    # {start, stop, times}: layers start .. stop-1 run `times` times in a row with the same weights
    # (every pass keeps a cache of its own); the learned vector 'loop.step'[t] is added to the
    # stream before pass t.
    loop: Optional[dict] = None
    residual_mult: float = 1.0     # "sandwich": both residual updates are multiplied by it

    @property
    def runs(self) -> List[tuple]:
        """The layers in the order they run: (layer, pass) pairs, pass None outside the repeated span."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None) for i in range(n)]
        a, b, t = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return ([(i, None) for i in range(a)] + [(i, p) for p in range(t) for i in range(a, b)]
                + [(i, None) for i in range(b, n)])

    @property
    def n_runs(self) -> int:
        return len(self.runs)

    def _validate_sandwich(self) -> None:
        for i, l in enumerate(self.layers):
            l.mixer.validate()
            if l.mixer.kind not in ("latent_attention", "softmax_attention"):
                raise ValueError(f"mixer {l.mixer.kind!r} does not belong to a 'sandwich' model")
            if l.mixer.kind == "latent_attention" and l.mixer.q_rank:
                raise ValueError("a 'sandwich' model's latent attention projects its queries straight from the input")
            src = l.mixer.kv_from
            if src >= 0:
                if self.loop is not None or l.mixer.kind != "softmax_attention" or not src < i:
                    raise ValueError(f"layer {i}: keys and values are read from an earlier softmax attention layer "
                                     "of a model without a repeated span")
                a, b = l.mixer, self.layers[src].mixer
                same = ("kind", "heads", "kv_heads", "dim", "vdim", "maps", "rot_dims", "rot_base", "rot_layout",
                        "rot_scaling", "qk_head_norm", "qk_full_norm")
                if b.kv_from >= 0 or b.value_is_key or any(getattr(a, k) != getattr(b, k) for k in same):
                    raise ValueError(f"layer {i}: layer {src} must project keys and values of its own, with this "
                                     "layer's head counts, sizes, norms and rotation")
            if l.ff < 0 or l.ff_act not in ("relu", "silu") or (l.ff and l.experts is not None):
                raise ValueError("a layer's feed-forward is gated (ff > 0, relu or silu) or routed experts, not both")
            if l.experts is not None:
                l.experts.validate()
        if self.loop is not None:
            a, b, t = (int(self.loop[k]) for k in ("start", "stop", "times"))
            if not 0 <= a < b <= len(self.layers) or t < 1:
                raise ValueError(f"loop {self.loop}: needs 0 <= start < stop <= layers and times >= 1")

    def validate(self) -> None:
        if self.width < 1 or self.vocab < 1 or not self.layers:
            raise ValueError("a model needs width, vocab and at least one layer")
        if self.block not in ("gated", "postnorm", "sandwich"):
            raise ValueError(f"unknown block {self.block!r}")
        if self.block == "sandwich":
            if self.bigram is not None:
                raise ValueError("a 'sandwich' model has no bigram table")
            return self._validate_sandwich()
        if self.loop is not None:
            raise ValueError("only a 'sandwich' model repeats a span of its layers")
        if self.bigram is not None and int(self.bigram["buckets"]) < 1:
            raise ValueError("a bigram table needs buckets >= 1")
        for l in self.layers:
            l.mixer.validate()
            if l.ff < 0:
                raise ValueError("ff must be >= 0")
            post = l.mixer.kind in ("latent_attention", "parallel")
            if post != (self.block == "postnorm"):
                raise ValueError(f"mixer {l.mixer.kind!r} does not belong to a {self.block!r} model")
            if l.experts is not None:
                l.experts.validate()
                if not post or l.ff:
                    raise ValueError("routed experts are the feed-forward of a postnorm layer, and its only one")
            elif post and l.ff:
                raise ValueError("a postnorm layer's feed-forward is a set of routed experts")

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def param_count(self) -> int:
        W, n = self.width, self.vocab * self.width + self.width
        if not self.tied_head:
            n += self.vocab * W
        if self.bigram:
            n += (int(self.bigram["buckets"]) + 1) * W
        if self.loop:
            n += int(self.loop["times"]) * W
        for l in self.layers:
            m = l.mixer
            if self.block == "sandwich":
                n += 2 * W + (2 * W if (l.ff or l.experts) else 0) + m.heads * m.vdim * W
                if m.kind == "latent_attention":
                    n += W * (m.heads * (m.dim + m.rot_dim) + m.kv_rank + m.rot_dim + (m.heads if m.head_gate else 0))
                    n += m.kv_rank + m.heads * (m.dim + m.vdim) * m.kv_rank + (m.heads if m.sink else 0)
                else:
                    nq, nk = m.heads * m.maps * m.dim, m.kv_heads * m.maps * m.dim
                    nv = 0 if m.value_is_key else m.kv_heads * m.vdim
                    n += W * nq + (0 if m.kv_from >= 0 else W * (nk + nv))
                    n += 2 * m.dim if m.qk_head_norm else ((nq + nk) if m.qk_full_norm else 0)
                    n += (nq + nk + W) if m.proj_bias else 0
                    n += 4 * m.dim if m.maps == 2 else 0
                n += 3 * l.ff * W
                ex = l.experts
                if ex is not None:
                    per = 3 if ex.act == "silu" else 2
                    n += ex.experts * (W + per * ex.ff * W) + per * ex.shared_ff * W
                    n += W if ex.shared_ff and ex.shared_gate else 0
                    n += ex.experts if ex.router_bias else 0
                continue
            if m.kind == "latent_attention":
                n += W + W * (m.q_rank + m.kv_rank + m.rot_dim) + m.q_rank + m.kv_rank
                n += m.heads * ((m.dim + m.rot_dim) * m.q_rank + (m.dim + m.vdim) * m.kv_rank + m.vdim * W)
            elif m.kind == "parallel":
                sd = m.ssd
                n += W + (W + 1) * (m.heads * m.dim + m.kv_heads * m.dim) + W * m.kv_heads * m.vdim + m.heads * m.vdim * W
                n += W * (2 * sd.inner + 2 * sd.groups * sd.state + sd.heads) + sd.conv_channels * (sd.taps + 1)
                n += 3 * sd.heads + sd.inner + sd.inner * W
            if l.experts is not None:
                n += W + l.experts.experts * (W + 3 * l.experts.ff * W)
            if m.kind in ("latent_attention", "parallel"):
                continue
            n += W + W * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim) + 2 * m.heads * m.vdim) + W * W + W
            n += (m.rank * (W + m.heads * m.dim) + m.heads * m.dim + m.vdim) if m.kind == "gla" else 0
            n += (3 * l.ff * W + W * W + W) if l.ff else 0
        return n

    def state_bytes_per_seq(self) -> int:
        n = 0
        for l in self.layers:
            m = l.mixer
            if m.kind == "parallel":
                n += 4 * (m.ssd.heads * m.ssd.state * m.ssd.vdim + (m.ssd.taps - 1) * m.ssd.conv_channels)
            elif m.kind in ("retention", "gla"):
                n += 4 * m.heads * m.dim * m.vdim
        return n


def puguzen_config(cfg: dict, tensor_shapes: Optional[dict] = None, **overrides) -> SeqModelConfig:
    """A Puguzen config.json.  tensor_shapes (name -> shape) supplies the sizes the file does not
    state (the inner size of a gla layer's low-rank pair)."""
    layers = []
    for i, l in enumerate(cfg["layers"]):
        m, kind = l["mixer"], l["type"]
        rot, mask = m.get("rot") or {}, m.get("mask") or {}
        rank = 0
        if kind == "gla":
            shape = (tensor_shapes or {}).get(f"l{i}.mix.a1")
            rank = int(shape[0]) if shape is not None else int(m.get("rank", 0))
        spec = MixerSpec(kind=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                         kv_heads=int(m.get("kv_heads", 0)), rot_dims=int(rot.get("dims", 0)),
                         rot_base=float(rot.get("base", 10000.0)),
                         rot_layout="interleaved" if kind == "attention" else "half",
                         decay=tuple(m["decay"]) if "decay" in m else None, tau=float(m.get("tau", 1.0)),
                         rank=rank, scale=float(m.get("scale", 1.0)), window=int(mask.get("size", 0)),
                         pool=int(mask.get("pool", 1)))
        mlp = l.get("mlp")
        if mlp and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported")
        layers.append(SeqLayerSpec(spec, int(mlp["ff"]) if mlp else 0))
    out = SeqModelConfig(arch="puguzen", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers,
                         norm_eps=float(cfg["norm"]["eps"]), name=cfg.get("architecture", "Puguzen"))
    for k, v in overrides.items():
        if not hasattr(out, k):
            raise ValueError(f"Unknown config parameter: {k}")
        setattr(out, k, v)
    out.validate()
    return out


def naburax_config(cfg: dict, tensor_shapes: Optional[dict] = None, **overrides) -> SeqModelConfig:
    """A Naburax config.json: latent-attention layers and layers with attention beside a
    state-space recurrence, in any order, each normed on its sublayers' outputs, routed experts
    as feed-forward, a scaled embedding plus a hashed table of token pairs, an untied head."""
    layers = []
    for i, l in enumerate(cfg["layers"]):
        m, kind = l["mixer"], l["type"]
        if kind == "latent_attention":
            rot = m.get("rot") or {}
            shape = (tensor_shapes or {}).get(f"l{i}.mix.dq")
            spec = MixerSpec(kind=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                             q_rank=int(shape[0]) if shape is not None else int(m["q_rank"]),
                             kv_rank=int(m["kv_rank"]), rot_dim=int(m.get("rot_dim", 0)),
                             rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                             rot_layout="interleaved", rot_scaling=rot.get("scaling") or None,
                             scale=float(m["scale"]), window=int(m["mask"]["size"]))
            if spec.q_rank < 1 or spec.window < 1:
                raise ValueError(f"layer {i}: latent attention needs a query latent and a window of at least one token")
        elif kind == "parallel":
            a, b = m["left"], m["right"]
            spec = MixerSpec(kind=kind, heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", 0)), dim=int(a["dim"]),
                             vdim=int(a["vdim"]), scale=float(a["scale"]), window=int(a["mask"]["size"]),
                             keep_first=int(a["mask"].get("keep_first", 0)),
                             ssd=SsdSpec(heads=int(b["heads"]), vdim=int(b["vdim"]), state=int(b["state"]),
                                         groups=int(b.get("groups", 1)), taps=int(b["conv"]),
                                         norm_groups=int(b.get("norm_groups", 1))),
                             left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = l.get("mlp")
        experts = None
        if mlp:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported")
            experts = ExpertsSpec(experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                                  ff=int(mlp["expert"]["ff"]))
        layers.append(SeqLayerSpec(spec, 0, experts))
    emb = cfg.get("embedding") or {}
    bg = emb.get("bigram")
    out = SeqModelConfig(arch="naburax", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers,
                         norm_eps=float(cfg["norm"]["eps"]), name=cfg.get("architecture", "Naburax"),
                         block="postnorm", embed_scale=float(emb.get("scale", 1.0)),
                         bigram={k: int(bg[k]) for k in ("buckets", "mul_prev", "mul_cur")} if bg else None,
                         tied_head=False, logit_scale=float(cfg.get("logit_scale", 1.0)))
    for k, v in overrides.items():
        if not hasattr(out, k):
            raise ValueError(f"Unknown config parameter: {k}")
        setattr(out, k, v)
    out.validate()
    return out


def fepopel_config(cfg: dict, tensor_shapes: Optional[dict] = None, **overrides) -> SeqModelConfig:
    """A Fepopel config.json: layers normed before and after each sublayer; latent attention over
    every earlier token (queries straight from the input, a learned sink per head in the softmax,
    outputs gated per head) and grouped-query softmax attention inside chunks (q and k normed per
    head, capped scores, no rotation), in any order; a gated feed-forward, routed experts of two
    matrices beside a gated shared expert, or none; a span of layers that runs several times over;
    a scaled embedding and an untied head."""
    layers = []
    for i, l in enumerate(cfg["layers"]):
        m, kind = l["mixer"], l["type"]
        if kind == "latent_attention":
            rot = m.get("rot") or {}
            rot_dim = int(m.get("rot_dim", 0))
            spec = MixerSpec(kind=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), q_rank=0,
                             kv_rank=int(m["kv_rank"]), rot_dim=rot_dim, rot_dims=int(rot.get("dims", rot_dim)),
                             rot_base=float(rot.get("base", 10000.0)), rot_layout="interleaved",
                             scale=float(m["scale"]), window=0, sink=True, head_gate=True)
        elif kind == "attention":
            mask = m.get("mask") or {}
            spec = MixerSpec(kind="softmax_attention", heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", 0)),
                             dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]), window=0,
                             chunk=int(mask.get("size") or 0), softcap=float(m.get("softcap") or 0.0), qk_head_norm=True)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = l.get("mlp")
        ff, experts = 0, None
        if mlp:
            mk = mlp.get("kind", "dense")
            if mk == "dense":
                ff = int(mlp["ff"])
            elif mk == "moe":
                r, sh = mlp["router"], mlp.get("shared")
                experts = ExpertsSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                                      score="softmax", renorm=True, scale_input=False, act="relu2", renorm_eps=1e-20,
                                      scale=float(r.get("scale", 1.0)), shared_ff=int(sh["ff"]) if sh else 0)
            else:
                raise ValueError(f"layer {i}: feed-forward kind {mk!r} is not supported")
        layers.append(SeqLayerSpec(spec, ff, experts, ff_act="silu"))
    emb, loop = cfg.get("embedding") or {}, cfg.get("loop")
    out = SeqModelConfig(arch="fepopel", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers,
                         norm_eps=float(cfg["norm"]["eps"]), name=cfg.get("architecture", "Fepopel"),
                         block="sandwich", embed_scale=float(emb.get("scale", 1.0)), tied_head=False,
                         loop={k: int(loop[k]) for k in ("start", "stop", "times")} if loop else None)
    for k, v in overrides.items():
        if not hasattr(out, k):
            raise ValueError(f"Unknown config parameter: {k}")
        setattr(out, k, v)
    out.validate()
    return out


def zopupel_config(cfg: dict, tensor_shapes: Optional[dict] = None, **overrides) -> SeqModelConfig:
    """A Zopupel config.json: layers normed before and after each sublayer, both residual updates
    multiplied by one constant; two causal grouped-query softmax attentions over every earlier
    token, in any order, with rotate-half rotary positions on the leading channels: "attention", a
    differential attention (two score maps per head, every frequency divided by a factor), which
    may read an earlier layer's cached keys and values (kv_from); "attention_2", whose values are
    its keys as projected, with biases on its projections, q and k normed over the whole
    projection, blended frequencies and one term of score 0 in the softmax's denominator.  Routed
    gated experts (a bias on the router, softmax over the chosen logits) beside an ungated shared
    expert, or no feed-forward; an untied head."""
    layers = []
    for i, l in enumerate(cfg["layers"]):
        m, kind = l["mixer"], l["type"]
        rot = m.get("rot") or {}
        common = dict(kind="softmax_attention", heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", 0)),
                      dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]), window=0,
                      rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_layout="half",
                      rot_scaling=rot.get("scaling") or None)
        if kind == "attention":
            src = m.get("kv_from")
            spec = MixerSpec(maps=2, diff=float(m["diff"]), kv_from=-1 if src is None else int(src), **common)
        elif kind == "attention_2":
            spec = MixerSpec(qk_full_norm=True, proj_bias=True, value_is_key=True, unit_sink=True, **common)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = l.get("mlp")
        experts = None
        if mlp:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported")
            r, sh = mlp["router"], mlp.get("shared")
            experts = ExpertsSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                                  score="softmax", renorm=True, scale_input=False, act="silu",
                                  shared_ff=int(sh["ff"]) if sh else 0, shared_gate=False, router_bias=True)
        layers.append(SeqLayerSpec(spec, 0, experts, ff_act="silu"))
    out = SeqModelConfig(arch="zopupel", width=int(cfg["width"]), vocab=int(cfg["vocab"]), layers=layers,
                         norm_eps=float(cfg["norm"]["eps"]), name=cfg.get("architecture", "Zopupel"),
                         block="sandwich", tied_head=False, residual_mult=float(cfg.get("residual_mult", 1.0)))
    for k, v in overrides.items():
        if not hasattr(out, k):
            raise ValueError(f"Unknown config parameter: {k}")
        setattr(out, k, v)
    out.validate()
    return out


# config.json "architecture" -> builder of a layer-list config
SEQ_ARCHITECTURES = {"Puguzen": puguzen_config, "Naburax": naburax_config, "Fepopel": fepopel_config,
                     "Zopupel": zopupel_config}


def safetensors_shapes(path: str) -> dict:
    """name -> shape from a safetensors file's header (8-byte length, then JSON)."""
    import struct
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in head.items() if k != "__metadata__"}


def load_model_config(model_dir: str, **overrides):
    """The configuration class a checkpoint folder asks for: a layer-list model if its
    config.json names one of SEQ_ARCHITECTURES, else a Hugging Face decoder (ModelConfig)."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    arch = cfg.get("architecture")
    if arch in SEQ_ARCHITECTURES:
        shapes = {}
        for fn in sorted(os.listdir(model_dir)):
            if fn.endswith(".safetensors"):
                shapes.update(safetensors_shapes(os.path.join(model_dir, fn)))
        return SEQ_ARCHITECTURES[arch](cfg, shapes, **overrides)
    if arch is not None and "model_type" not in cfg:
        raise ValueError(f"unknown architecture {arch!r}; known: {sorted(SEQ_ARCHITECTURES)}")
    return from_hf_config(cfg, **overrides)
