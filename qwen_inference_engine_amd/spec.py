"""Model specs (replace the reference's hard-coded Qwen3-14B dims).

Reference literals: layers/src/utills.cu:8-16 (dims), layers/include/iengine.cuh:19-21
(CONTEXT_SIZE, HIDDEN_DIM_KV, NUM_OF_LAYERS), normalization.cu:9 / qk_norm.cu:46 (eps 1e-4),
include.cpp:7 (RoPE base 1e6).  In ``ref`` numerics the reference's eps/base are used for
every model (they are op semantics of the reference engine); ``hf`` numerics take the
model's own config values.
"""
from __future__ import annotations

import dataclasses
import json

from typing import List, Optional, Tuple

from . import _lib
from ._lib import ModelSpecC, QIE_NUMERICS_HF, QIE_NUMERICS_REF

REF_EPS = 1e-4        # normalization.cu:9, qk_norm.cu:46
REF_THETA = 1e6       # include.cpp:7


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    name: str
    n_layers: int
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    ffn: int
    vocab: int
    tie_embeddings: bool
    qkv_bias: bool
    qk_norm: bool
    hf_eps: float
    hf_theta: float = 1e6
    numerics: str = "ref"

    @property
    def rms_eps(self) -> float:
        return REF_EPS if self.numerics == "ref" else self.hf_eps

    @property
    def rope_theta(self) -> float:
        return REF_THETA if self.numerics == "ref" else self.hf_theta

    @property
    def q_dim(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim

    def with_numerics(self, numerics: str) -> "ModelSpec":
        assert numerics in ("ref", "hf")
        return dataclasses.replace(self, numerics=numerics)

    def replace(self, **kw) -> "ModelSpec":
        return dataclasses.replace(self, **kw)

    def to_c(self) -> ModelSpecC:
        s = ModelSpecC()
        s.n_layers, s.hidden, s.n_heads = self.n_layers, self.hidden, self.n_heads
        s.n_kv_heads, s.head_dim, s.ffn, s.vocab = self.n_kv_heads, self.head_dim, self.ffn, self.vocab
        s.tie_embeddings, s.qkv_bias, s.qk_norm = int(self.tie_embeddings), int(self.qkv_bias), int(self.qk_norm)
        s.rms_eps, s.rope_theta = self.rms_eps, self.rope_theta
        s.numerics = QIE_NUMERICS_REF if self.numerics == "ref" else QIE_NUMERICS_HF
        return s

    # ------------------------------------------------------------ accounting
    def layer_weight_bytes(self) -> int:
        H, I = self.hidden, self.ffn
        n = (self.q_dim + 2 * self.kv_dim) * H + H * self.q_dim + 3 * H * I + 2 * H
        if self.qkv_bias:
            n += self.q_dim + 2 * self.kv_dim
        if self.qk_norm:
            n += 2 * self.head_dim
        return 2 * n

    def decode_weight_bytes(self, fp8: bool = False) -> int:
        """Weights streamed per decode step: every layer + final norm + lm_head once.
        fp8: linear weights and lm_head at 1 byte per weight + one fp32 scale per row."""
        if not fp8:
            return self.n_layers * self.layer_weight_bytes() + 2 * self.hidden + 2 * self.vocab * self.hidden
        lin = self.linear_params_per_layer()
        rows = self.q_dim + 2 * self.kv_dim + self.hidden + 2 * self.ffn + self.hidden
        other = self.layer_weight_bytes() - 2 * lin            # norms, biases (bf16)
        per_layer = lin + 4 * rows + other
        return self.n_layers * per_layer + 2 * self.hidden + (self.vocab * self.hidden + 4 * self.vocab)

    def kv_bytes_per_position(self) -> int:
        return self.n_layers * 2 * self.kv_dim * 2

    def linear_params_per_layer(self) -> int:
        H, I = self.hidden, self.ffn
        return (self.q_dim + 2 * self.kv_dim) * H + H * self.q_dim + 3 * H * I

    def prefill_flops(self, P: int, B: int = 1) -> float:
        lin = 2.0 * P * B * self.n_layers * self.linear_params_per_layer()
        attn = self.n_layers * 4.0 * self.q_dim * P * (P + 1) / 2 * B
        head = 2.0 * self.hidden * self.vocab * B
        return lin + attn + head

    @classmethod
    def from_hf_config(cls, cfg: dict, name: str = "hf", numerics: str = "ref") -> "ModelSpec":
        hd = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
        mt = cfg.get("model_type", "qwen2")
        return cls(name=name, n_layers=cfg["num_hidden_layers"], hidden=cfg["hidden_size"],
                   n_heads=cfg["num_attention_heads"], n_kv_heads=cfg["num_key_value_heads"],
                   head_dim=hd, ffn=cfg["intermediate_size"], vocab=cfg["vocab_size"],
                   tie_embeddings=bool(cfg.get("tie_word_embeddings", False)),
                   qkv_bias=(mt == "qwen2") or bool(cfg.get("attention_bias", False)),
                   qk_norm=(mt == "qwen3"), hf_eps=float(cfg.get("rms_norm_eps", 1e-6)),
                   hf_theta=float(cfg.get("rope_theta", 1e6)), numerics=numerics)

    @classmethod
    def from_json(cls, path: str, numerics: str = "ref") -> "ModelSpec":
        with open(path) as f:
            return cls.from_hf_config(json.load(f), name=path, numerics=numerics)


QWEN2_0_5B = ModelSpec("Qwen2-0.5B", 24, 896, 14, 2, 64, 4864, 151936, True, True, False, 1e-6)
QWEN2_7B = ModelSpec("Qwen2-7B", 28, 3584, 28, 4, 128, 18944, 152064, False, True, False, 1e-6)
QWEN2_72B = ModelSpec("Qwen2-72B", 80, 8192, 64, 8, 128, 29568, 152064, False, True, False, 1e-5)
QWEN3_14B = ModelSpec("Qwen3-14B", 40, 5120, 40, 8, 128, 17408, 151936, False, False, True, 1e-6)

PRESETS = {s.name: s for s in (QWEN2_0_5B, QWEN2_7B, QWEN2_72B, QWEN3_14B)}


def tiny(name: str = "tiny-qwen2", *, n_layers=2, hidden=128, n_heads=4, n_kv_heads=2, head_dim=64,
         ffn=256, vocab=512, tie=False, bias=True, qk_norm=False, numerics="ref") -> ModelSpec:
    """Small test configurations (oracle finishes in well under a second)."""
    return ModelSpec(name, n_layers, hidden, n_heads, n_kv_heads, head_dim, ffn, vocab, tie, bias,
                     qk_norm, 1e-6, 1e6, numerics)


def shard_heads(nq: int, nkv: int, tp: int, rank: int):
    """(local q heads, first q head, local kv heads, first kv head) of `rank` — the rule of
    engine.hip shard_heads: even split when tp divides the kv heads, else every kv head on
    tp / nkv ranks that split its group's q heads (the first G % rep ranks one more);
    None when the heads do not shard."""
    if nkv % tp == 0 and nq % tp == 0:
        return nq // tp, rank * (nq // tp), nkv // tp, rank * (nkv // tp)
    if tp % nkv:
        return None
    rep, G = tp // nkv, nq // nkv
    if rep > G:
        return None
    g, sub = rank // rep, rank % rep
    base, extra = G // rep, G % rep
    return base + (1 if sub < extra else 0), g * G + sub * base + min(sub, extra), 1, g


def tp_shardable(spec: ModelSpec, tp: int):
    """(ok, reason): can `spec` run tensor-parallel over `tp` ranks (qie_engine_create's check)?"""
    if shard_heads(spec.n_heads, spec.n_kv_heads, tp, 0) is None:
        return False, f"{spec.n_heads} q / {spec.n_kv_heads} kv heads do not shard {tp} ways"
    if spec.ffn % tp or (spec.ffn // tp) % 8:
        return False, f"ffn {spec.ffn} / {tp} is not a multiple of 8"
    if spec.vocab % tp:
        return False, f"vocab {spec.vocab} not divisible by {tp}"
    return True, ""


# ------------------------------------------------------------------ layered models
# Models given as a list of layers, each with its own mixer and feed-forward (the engine tier of
# qie_engine_create_layered).  A config.json of such a model names its design in "architecture";
# ARCHITECTURES maps that name to the reader of the config.

@dataclasses.dataclass(frozen=True)
class LatentAttention:
    """Mixer: latent (compressed-KV) attention, causal or over a sliding window; options: a per-head
    output gate, queries through a latent of their own, either rotary pairing, scaled frequencies."""
    heads: int
    dim: int          # unrotated query / key coordinates per head
    rot_dim: int      # rotated coordinates per head (the key's are shared by all heads)
    vdim: int
    kv_rank: int
    window: int
    rot_dims: int     # rotated coordinates that actually turn (rotate-half pairs i, i + rot_dims / 2)
    rot_base: float
    scale: float
    kv_from: Optional[int] = None   # the layer whose cache rows this layer reads
    q_rank: int = 0                 # > 0: q = W_uq rms(W_dq x) w through a latent of this size (no W_q)
    rot_layout: str = "halves"      # "halves" | "interleaved"
    head_gate: bool = True          # head h's output times sigmoid(W_g x)_h
    rot_scaling: Optional[Tuple[float, float, float, float]] = None   # (factor, low, high, original)


@dataclasses.dataclass(frozen=True)
class GqaAttention:
    """Mixer: grouped-query softmax attention over a paged K / V cache; every option is a field
    (qie_gqa_desc): head norms, rotary pairing and extent, turned values, mask, keys as values,
    log-distance bias."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    qk_norm: str = "none"        # "none" | "weight" | "plain"
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_layout: str = "halves"   # "halves" (i, i + dims/2) | "interleaved" (2i, 2i + 1)
    rot_values: bool = False
    mask: str = "causal"         # "causal" | "window" | "chunk"
    mask_size: int = 0
    values_are_keys: bool = False
    dist_bias: bool = False
    weights: str = "softmax"     # "softmax" | "sigmoid": sigmoid(score + a number per head), not normalised
    slope_bias: bool = False     # the score loses 2^(-8 (h + 1) / heads) * (i - j)
    head_gate: bool = False      # head h's output times sigmoid(W_g x)_h
    q_temp_coef: float = 0.0     # q times 1 + coef * ln(floor((pos + 1) / every) + 1) after its norm
    q_temp_every: int = 0        # 0: no query temperature
    qk_bias: bool = False        # bias vectors on the q and k projections
    sink: bool = False           # exp(a number per head) joins the softmax denominator
    out_gate: bool = False       # the concatenated head outputs times sigmoid(W_g x), element by element
    rot_scaling: Optional[Tuple[float, float, float, float]] = None   # (factor, low, high, original) wavelengths


@dataclasses.dataclass(frozen=True)
class GatedRecurrence:
    """Gated linear recurrence (HGRN2 form): a [dim, vdim] fp32 state per head and slot."""
    heads: int
    dim: int
    vdim: int


@dataclasses.dataclass(frozen=True)
class AttentionWithRecurrence:
    """Mixer: a GqaAttention and a GatedRecurrence read the same input; their results are added
    with fixed scales."""
    attn: GqaAttention
    rec: GatedRecurrence
    attn_scale: float
    rec_scale: float


@dataclasses.dataclass(frozen=True)
class MinGru:
    """Mixer: minGRU, a recurrence per channel whose update gate and candidate depend on the current input alone; `width` fp32 state
    elements per slot."""
    width: int


@dataclasses.dataclass(frozen=True)
class ChannelDelta:
    """Mixer: gated delta rule with one decay per head and key channel; short convolutions on q, k, v;
    a [dim, vdim] fp32 state per head and slot plus the convolutions' last inputs."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int         # taps of the short convolutions
    rank_a: int       # rows of W_a1 (decay) and W_g1 (output gate)
    rank_g: int

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim


@dataclasses.dataclass(frozen=True)
class FeedForward:
    kind: str         # "dense" or "moe"
    ff: int           # hidden size (of one expert for "moe")
    experts: int = 0
    top: int = 0
    router: str = "sigmoid_in"   # "sigmoid_in": sigmoid scores scale the input; "softmax_out":
                                 # biased logits, softmax over the chosen ones weights the output;
                                 # "softmax_all": softmax over all router outputs, chosen by score +
                                 # correction inside the best groups, renormalised, times route_scale
    act: str = "silu_gated"      # dense: "silu_gated" | "gelu_tanh_gated" (gate, up, down) | "xielu" (up, down, two numbers)
    identity: int = 0            # "softmax_all": identity experts after the `experts` real ones
    groups: int = 1
    groups_keep: int = 1
    route_scale: float = 1.0


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    mixer: object     # LatentAttention | GqaAttention | AttentionWithRecurrence | MinGru | ChannelDelta
    mlp: Optional[FeedForward]


@dataclasses.dataclass(frozen=True)
class LayeredSpec:
    name: str
    width: int
    vocab: int
    norm_eps: float
    layers: Tuple[LayerSpec, ...]
    depth_mix: bool = True
    block: str = "postnorm_gain"     # "postnorm_gain" | "sandwich" (weight-vector norms around every branch)
                                     # | "prenorm" (one plain-weight norm before every branch)
    tied_head: bool = False
    embed_scale: float = 1.0
    pos_embed: str = "none"          # "none" | "sinusoid" (added to the scaled embedding row)
    loop: Optional[Tuple[int, int, int]] = None   # (start, stop, times): layers [start, stop) run `times` times
    # pre-norm block options
    norm_offset: float = 0.0         # norm weights are norm_offset + w (1: stored around zero)
    streams: int = 0                 # >= 1: that many residual rows mixed by 'l<i>.hc<q>.in|out|mix' (hyper-connections)
    canon_taps: int = 0              # >= 1: the mixer reads h + causal conv(h) over time ('l<i>.canon1' [width, taps])
    embed_norm: bool = False         # the embedding rows are normed with 'embed.norm'

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> List[int]:
        """Layer index of every layer run, in execution order."""
        n = len(self.layers)
        if not self.loop or self.loop[2] <= 1 or self.loop[1] <= self.loop[0]:
            return list(range(n))
        a, b, t = self.loop
        return list(range(a)) + list(range(a, b)) * t + list(range(b, n))

    @property
    def n_runs(self) -> int:
        return len(self.runs())

    @property
    def hidden(self) -> int:
        return self.width

    def to_c(self):
        """(ArchDescC, keepalive of its layer array)."""
        arr = (_lib.LayerDescC * len(self.layers))()
        def gqa(g, m):
            g.heads, g.kv_heads, g.dim, g.vdim, g.scale = m.heads, m.kv_heads, m.dim, m.vdim, m.scale
            g.qk_norm = {"none": _lib.QIE_QKNORM_NONE, "weight": _lib.QIE_QKNORM_WEIGHT, "plain": _lib.QIE_QKNORM_PLAIN}[m.qk_norm]
            g.rot_dims, g.rot_base = m.rot_dims, m.rot_base
            g.rot_layout = {"halves": _lib.QIE_ROT_HALVES, "interleaved": _lib.QIE_ROT_INTERLEAVED}[m.rot_layout]
            g.rot_values = int(m.rot_values)
            g.mask = {"causal": _lib.QIE_MASK_CAUSAL, "window": _lib.QIE_MASK_WINDOW, "chunk": _lib.QIE_MASK_CHUNK}[m.mask]
            g.mask_size, g.values_are_keys, g.dist_bias = m.mask_size, int(m.values_are_keys), int(m.dist_bias)
            g.weights = _lib.QIE_WEIGHTS_SIGMOID if m.weights == "sigmoid" else _lib.QIE_WEIGHTS_SOFTMAX
            g.slope_bias, g.head_gate = int(m.slope_bias), int(m.head_gate)
            g.q_temp_coef, g.q_temp_every = m.q_temp_coef, m.q_temp_every
            g.qk_bias, g.sink, g.out_gate = int(m.qk_bias), int(m.sink), int(m.out_gate)
            if m.rot_scaling:
                g.rot_scaling.factor, g.rot_scaling.low, g.rot_scaling.high, g.rot_scaling.original = m.rot_scaling

        for d, L in zip(arr, self.layers):
            m = L.mixer
            if isinstance(m, GqaAttention):
                d.mixer = _lib.QIE_MIXER_GQA
                gqa(d.gqa, m)
            elif isinstance(m, AttentionWithRecurrence):
                d.mixer = _lib.QIE_MIXER_GQA_RECURRENT
                gqa(d.gqa, m.attn)
                d.rec.heads, d.rec.dim, d.rec.vdim = m.rec.heads, m.rec.dim, m.rec.vdim
                d.gqa_scale, d.rec_scale = m.attn_scale, m.rec_scale
            elif isinstance(m, MinGru):
                d.mixer = _lib.QIE_MIXER_MINGRU
                d.mingru.width = m.width
            elif isinstance(m, ChannelDelta):
                d.mixer = _lib.QIE_MIXER_CHANNEL_DELTA
                x = d.delta
                x.heads, x.kv_heads, x.dim, x.vdim, x.conv, x.rank_a, x.rank_g = m.heads, m.kv_heads, m.dim, m.vdim, m.conv, m.rank_a, m.rank_g
            else:
                d.mixer = _lib.QIE_MIXER_LATENT_ATTENTION
                d.heads, d.dim, d.rot_dim, d.vdim, d.kv_rank = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
                d.window, d.kv_from, d.rot_dims = m.window, -1 if m.kv_from is None else m.kv_from, m.rot_dims
                d.rot_base, d.scale = m.rot_base, m.scale
                d.q_rank, d.head_gate = m.q_rank, int(m.head_gate)
                d.rot_layout = {"halves": _lib.QIE_ROT_HALVES, "interleaved": _lib.QIE_ROT_INTERLEAVED}[m.rot_layout]
                if m.rot_scaling:
                    d.rot_scaling.factor, d.rot_scaling.low, d.rot_scaling.high, d.rot_scaling.original = m.rot_scaling
            if L.mlp is None:
                d.ff_kind = _lib.QIE_FF_NONE
            elif L.mlp.kind == "dense":
                d.ff_kind, d.ff = _lib.QIE_FF_DENSE, L.mlp.ff
                d.ff_act = {"silu_gated": _lib.QIE_ACT_SILU_GATED, "xielu": _lib.QIE_ACT_XIELU,
                            "gelu_tanh_gated": _lib.QIE_ACT_GELU_TANH_GATED}[L.mlp.act]
            else:
                d.ff_kind, d.ff, d.experts, d.top = _lib.QIE_FF_MOE, L.mlp.ff, L.mlp.experts, L.mlp.top
                d.router = {"sigmoid_in": _lib.QIE_ROUTER_SIGMOID_IN, "softmax_out": _lib.QIE_ROUTER_SOFTMAX_OUT,
                            "softmax_all": _lib.QIE_ROUTER_SOFTMAX_ALL}[L.mlp.router]
                d.identity, d.groups, d.groups_keep, d.route_scale = L.mlp.identity, L.mlp.groups, L.mlp.groups_keep, L.mlp.route_scale
        a = _lib.ArchDescC()
        a.n_layers, a.width, a.vocab, a.norm_eps = len(self.layers), self.width, self.vocab, self.norm_eps
        a.depth_mix = int(self.depth_mix)
        a.block = {"postnorm_gain": _lib.QIE_BLOCK_POSTNORM_GAIN, "sandwich": _lib.QIE_BLOCK_SANDWICH,
                   "prenorm": _lib.QIE_BLOCK_PRENORM}[self.block]
        a.tied_head = int(self.tied_head)
        a.embed_scale = self.embed_scale
        a.pos_embed = _lib.QIE_POS_SINUSOID if self.pos_embed == "sinusoid" else _lib.QIE_POS_NONE
        if self.loop:
            a.loop_start, a.loop_stop, a.loop_times = self.loop
        a.layers = arr
        a.streams, a.canon_taps, a.embed_norm, a.norm_offset = self.streams, self.canon_taps, int(self.embed_norm), self.norm_offset
        return a, arr

    def tensor_shapes(self) -> "dict[str, List[int]]":
        """Checkpoint tensor names and shapes of this architecture."""
        W, out = self.width, {"embed": [self.vocab, self.width]}
        sandwich = self.block == "sandwich"
        nshape = [W] if self.block in ("sandwich", "prenorm") else []

        def gqa(q, m):
            out[q + "q"], out[q + "k"] = [m.heads * m.dim, W], [m.kv_heads * m.dim, W]
            if not m.values_are_keys:
                out[q + "v"] = [m.kv_heads * m.vdim, W]
            if m.qk_norm == "weight":
                out[q + "q.norm"], out[q + "k.norm"] = [m.dim], [m.dim]
            if m.dist_bias:
                out[q + "r1"], out[q + "r2"] = [m.heads], [m.heads]
            if m.weights == "sigmoid":
                out[q + "pb"] = [m.heads]
            if m.head_gate:
                out[q + "g"] = [m.heads, W]
            if m.qk_bias:
                out[q + "q.b"], out[q + "k.b"] = [m.heads * m.dim], [m.kv_heads * m.dim]
            if m.sink:
                out[q + "sink"] = [m.heads]
            if m.out_gate:
                out[q + "g"] = [m.heads * m.vdim, W]
            out[q + "o"] = [W, m.heads * m.vdim]

        if self.embed_norm:
            out["embed.norm"] = [W]
        for i, L in enumerate(self.layers):
            m, p = L.mixer, f"l{i}."
            for q in (("hc1.", "hc2.") if L.mlp is not None else ("hc1.",)) if self.streams else ():
                out[p + q + "in"], out[p + q + "out"], out[p + q + "mix"] = [self.streams], [self.streams], [self.streams, self.streams]
            if self.canon_taps:
                out[p + "canon1"] = [W, self.canon_taps]
            out[p + "norm1"] = nshape
            if sandwich:
                out[p + "norm1b"] = nshape
            if L.mlp is not None:
                out[p + "norm2"] = nshape
                if sandwich:
                    out[p + "norm2b"] = nshape
            if isinstance(m, GqaAttention):
                gqa(p + "mix.", m)
            elif isinstance(m, AttentionWithRecurrence):
                gqa(p + "mix.left.", m.attn)
                r, c = p + "mix.right.", m.rec
                out[r + "q"], out[r + "f"], out[r + "v"] = [c.heads * c.dim, W], [c.heads * c.dim, W], [c.heads * c.vdim, W]
                out[r + "f.b"], out[r + "lower"], out[r + "norm"] = [c.heads * c.dim], [c.heads * c.dim], [c.vdim]
                out[r + "o"] = [W, c.heads * c.vdim]
            elif isinstance(m, MinGru):
                q = p + "mix."
                out.update({q + "z": [m.width, W], q + "z.b": [m.width], q + "x": [m.width, W], q + "x.b": [m.width],
                            q + "g": [m.width, W], q + "o": [W, m.width]})
            elif isinstance(m, ChannelDelta):
                q = p + "mix."
                nk, nv = m.kv_heads * m.dim, m.heads * m.vdim
                out.update({q + "q": [nk, W], q + "q.conv": [nk, m.conv], q + "k": [nk, W], q + "k.conv": [nk, m.conv],
                            q + "v": [nv, W], q + "v.conv": [nv, m.conv], q + "b": [m.heads, W], q + "A_log": [m.heads],
                            q + "norm": [m.vdim], q + "a1": [m.rank_a, W], q + "a2": [m.heads * m.dim, m.rank_a],
                            q + "dt_bias": [m.heads * m.dim], q + "g1": [m.rank_g, W], q + "g2": [nv, m.rank_g], q + "o": [W, nv]})
            elif m.q_rank > 0:
                out[p + "mix.dq"], out[p + "mix.dq.norm"] = [m.q_rank, W], [m.q_rank]
                out[p + "mix.uq"] = [m.heads * (m.dim + m.rot_dim), m.q_rank]
            else:
                out[p + "mix.q"] = [m.heads * (m.dim + m.rot_dim), W]
            if isinstance(m, LatentAttention):
                if m.kv_from is None:
                    out[p + "mix.dkv"] = [m.kv_rank + m.rot_dim, W]
                    out[p + "mix.dkv.norm"] = [m.kv_rank]
                out[p + "mix.uk"] = [m.heads * m.dim, m.kv_rank]
                out[p + "mix.uv"] = [m.heads * m.vdim, m.kv_rank]
                if m.head_gate:
                    out[p + "mix.g"] = [m.heads, W]
                out[p + "mix.o"] = [W, m.heads * m.vdim]
            if L.mlp is not None and L.mlp.kind == "dense" and L.mlp.act == "xielu":
                out.update({p + "mlp.up": [L.mlp.ff, W], p + "mlp.down": [W, L.mlp.ff], p + "mlp.act": [2]})
            elif L.mlp is not None and L.mlp.kind == "dense":
                out.update({p + "mlp.gate": [L.mlp.ff, W], p + "mlp.up": [L.mlp.ff, W], p + "mlp.down": [W, L.mlp.ff]})
            elif L.mlp is not None:
                for e in range(L.mlp.experts):
                    q = f"{p}mlp.e{e}."
                    out.update({q + "gate": [L.mlp.ff, W], q + "up": [L.mlp.ff, W], q + "down": [W, L.mlp.ff]})
                out[p + "mlp.router"] = [L.mlp.experts + L.mlp.identity, W]
                if L.mlp.router == "softmax_out":
                    out[p + "mlp.router.b"] = [L.mlp.experts]
                if L.mlp.router == "softmax_all":
                    out[p + "mlp.correction"] = [L.mlp.experts + L.mlp.identity]
            if self.depth_mix:
                out[p + "dwa"] = [i + 2]
        out["final.norm"] = nshape
        if not self.tied_head:
            out["head"] = [self.vocab, W]
        return out

    def cache_row_elems(self) -> int:
        """Cached elements per token, all layer runs together."""
        n = 0
        for i in self.runs():
            m = self.layers[i].mixer
            if isinstance(m, LatentAttention):
                n += m.kv_rank + m.rot_dim if m.kv_from is None else 0
            elif isinstance(m, (MinGru, ChannelDelta)):
                pass
            else:
                a = m.attn if isinstance(m, AttentionWithRecurrence) else m
                n += a.kv_heads * (a.dim + a.vdim)
        return n

    def state_elems(self) -> int:
        """fp32 state elements per slot (recurrent mixers), all layer runs together."""
        n = 0
        for i in self.runs():
            m = self.layers[i].mixer
            if isinstance(m, AttentionWithRecurrence):
                n += m.rec.heads * m.rec.dim * m.rec.vdim
            elif isinstance(m, MinGru):
                n += m.width
            elif isinstance(m, ChannelDelta):
                n += m.heads * m.dim * m.vdim + (m.conv - 1) * m.conv_channels
            if self.canon_taps > 1:
                n += (self.canon_taps - 1) * self.width
        return n

    def step_flops(self, rows: int, ctx: int) -> float:
        """Multiply-adds x 2 of one step of `rows` tokens whose windows hold about `ctx` keys."""
        W, f = self.width, 0.0
        for i in self.runs():
            L = self.layers[i]
            m = L.mixer
            if isinstance(m, ChannelDelta):
                nk, nv = m.kv_heads * m.dim, m.heads * m.vdim
                f += 2.0 * rows * W * (2 * nk + 2 * nv + m.heads + m.rank_a + m.rank_g)
                f += 2.0 * rows * (m.rank_a * m.heads * m.dim + m.rank_g * nv) + 2.0 * rows * m.heads * m.dim * m.vdim * 3
                if L.mlp is not None:
                    f += 2.0 * rows * 3 * W * L.mlp.ff
                continue
            if isinstance(m, MinGru):
                f += 2.0 * rows * W * 4 * m.width
                if L.mlp is not None:
                    f += 2.0 * rows * (1 if L.mlp.kind == "dense" else L.mlp.top) * (2 if L.mlp.act == "xielu" else 3) * W * L.mlp.ff
                continue
            if not isinstance(m, LatentAttention):
                a = m.attn if isinstance(m, AttentionWithRecurrence) else m
                n_in = a.heads * a.dim + a.kv_heads * (a.dim + (0 if a.values_are_keys else a.vdim)) + (a.heads if a.head_gate else 0) \
                    + (a.heads * a.vdim if a.out_gate else 0)
                n_cat = a.heads * a.vdim
                keys = ctx if a.mask == "causal" else min(ctx, a.mask_size if a.mask == "window" else (a.mask_size + 1) // 2)
                f += 2.0 * rows * a.heads * keys * (a.dim + a.vdim)
                if isinstance(m, AttentionWithRecurrence):
                    c = m.rec
                    n_in += c.heads * (2 * c.dim + c.vdim)
                    n_cat += c.heads * c.vdim
                    f += 2.0 * rows * c.heads * c.dim * c.vdim * 2
                f += 2.0 * rows * W * (n_in + n_cat)
                if L.mlp is not None:
                    f += 2.0 * rows * (1 if L.mlp.kind == "dense" else L.mlp.top) * (2 if L.mlp.act == "xielu" else 3) * W * L.mlp.ff
                continue
            n_in = (m.heads * (m.dim + m.rot_dim) if m.q_rank == 0 else m.q_rank) + (m.heads if m.head_gate else 0) \
                + (m.kv_rank + m.rot_dim if m.kv_from is None else 0)
            f += 2.0 * rows * m.q_rank * m.heads * (m.dim + m.rot_dim)
            f += 2.0 * rows * W * n_in + 2.0 * rows * m.heads * m.kv_rank * (m.dim + m.vdim) + 2.0 * rows * W * m.heads * m.vdim
            f += 2.0 * rows * m.heads * (min(ctx, m.window) if m.window > 0 else ctx) * (2 * m.kv_rank + m.rot_dim)
            if L.mlp is not None:
                k = 1 if L.mlp.kind == "dense" else L.mlp.top
                f += 2.0 * rows * k * 3 * W * L.mlp.ff
        return f + 2.0 * rows * W * self.vocab


def _tivazen_from_config(cfg: dict, name: str) -> LayeredSpec:
    layers = []
    for i, L in enumerate(cfg["layers"]):
        if L["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        m = L["mixer"]
        rot = m.get("rot") or {}
        mixer = LatentAttention(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), window=int(m["mask"]["size"]), rot_dims=int(rot.get("dims", m["rot_dim"])),
            rot_base=float(rot.get("base", 10000.0)), scale=float(m["scale"]),
            kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))
        f = L.get("mlp")
        if f is None:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForward("dense", int(f["ff"]))
        elif f["kind"] == "moe":
            mlp = FeedForward("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]))
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mixer, mlp))
    return LayeredSpec(name, int(cfg["width"]), int(cfg["vocab"]), float(cfg["norm"]["eps"]), tuple(layers), True)


def _nodutar_from_config(cfg: dict, name: str) -> LayeredSpec:
    """Nodutar: sandwich-normed blocks whose mixer is either a block-local grouped-query attention
    (normed, partly rotated queries and keys, values turned by their position) beside a gated
    linear recurrence, or a causal attention whose values are its keys and whose scores carry a
    log-distance bias; softmax-routed experts; an optional repeated group of layers; tied head."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] == "parallel":
            a, c = m["left"], m["right"]
            attn = GqaAttention(
                heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]), scale=float(a["scale"]),
                qk_norm="weight", rot_dims=int(a["rot"]["dims"]), rot_base=float(a["rot"]["base"]), rot_layout="interleaved",
                rot_values=True, mask="chunk", mask_size=int(a["mask"]["size"]))
            rec = GatedRecurrence(heads=int(c["heads"]), dim=int(c["dim"]), vdim=int(c["vdim"]))
            mixer = AttentionWithRecurrence(attn, rec, float(m["left_scale"]), float(m["right_scale"]))
        elif L["type"] == "attention":
            mixer = GqaAttention(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["dim"]),
                                 scale=float(m["scale"]), qk_norm="plain", mask="causal", values_are_keys=True, dist_bias=True)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        f = L.get("mlp")
        if f is None:
            mlp = None
        elif f["kind"] == "moe":
            mlp = FeedForward("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]), "softmax_out")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mixer, mlp))
    lp = cfg.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None
    if loop and not (0 <= loop[0] <= loop[1] <= len(layers) and loop[2] >= 1):
        raise ValueError(f"loop {loop} does not fit {len(layers)} layers")
    return LayeredSpec(name, int(cfg["width"]), int(cfg["vocab"]), float(cfg["norm"]["eps"]), tuple(layers), depth_mix=False,
                       block="sandwich", tied_head=True, loop=loop)


def _lugipel_from_config(cfg: dict, name: str) -> LayeredSpec:
    """Lugipel: pre-normed blocks (plain-weight RMS norms) over a scaled embedding with a sinusoidal
    position vector.  Mixers: a sliding-window grouped-query attention without rotation (normed
    queries and keys, a query temperature that grows with the position, a linear distance bias with
    fixed head slopes, sigmoid weights with a bias per head instead of a softmax, a sigmoid gate per
    head) or a minGRU recurrence.  Feed-forward: dense with the xIELU activation, or gated-SiLU
    experts (some of them identity experts) routed by a softmax over all of them with a correction
    for the choice, group-limited, renormalised and scaled.  Untied head."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        if L["type"] == "attention":
            qt = m.get("q_temp") or {}
            mixer = GqaAttention(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                qk_norm="weight", mask="window", mask_size=int(m["mask"]["size"]), weights="sigmoid", slope_bias=True, head_gate=True,
                q_temp_coef=float(qt.get("coef", 0.0)), q_temp_every=int(qt.get("every", 0)))
        elif L["type"] == "mingru":
            mixer = MinGru(width=int(m["width"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        f = L.get("mlp")
        if f is None:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForward("dense", int(f["ff"]), act="xielu")
        elif f["kind"] == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            mlp = FeedForward("moe", int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), "softmax_all",
                              identity=int(r.get("identity", 0)), groups=int(g.get("count", 1)), groups_keep=int(g.get("keep", 1)),
                              route_scale=float(r.get("scale", 1.0)))
            n = mlp.experts + mlp.identity
            if mlp.groups < 1 or n % mlp.groups or not 1 <= mlp.groups_keep <= mlp.groups:
                raise ValueError(f"layer {i}: {n} router outputs do not form {mlp.groups} equal groups (keep {mlp.groups_keep})")
            if mlp.top > mlp.groups_keep * (n // mlp.groups):
                raise ValueError(f"layer {i}: top {mlp.top} above the {mlp.groups_keep} kept groups' experts")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mixer, mlp))
    return LayeredSpec(name, int(cfg["width"]), int(cfg["vocab"]), float(cfg["norm"]["eps"]), tuple(layers), depth_mix=False,
                       block="prenorm", tied_head=False, embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                       pos_embed="sinusoid")


def _rot_scaling(rot: dict):
    sc = rot.get("scaling")
    if not sc:
        return None
    t = (float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
    if not (t[0] > 0 and t[2] > t[1] >= 0 and t[3] > 0):
        raise ValueError(f"rotary scaling {sc}: factor and original must be positive, high above low")
    return t


def _verelorn_from_config(cfg: dict, name: str) -> LayeredSpec:
    """Verelorn: pre-normed blocks (RMS norms with weights stored around zero, also on the embedding rows)
    over several residual streams mixed by learned hyper-connections; the mixer reads its normed input
    plus a short causal convolution of it.  Mixers: a causal grouped-query attention whose values are
    its keys as projected (biased q / k, partial rotate-half rotary with wavelength-scaled frequencies,
    a sink in the softmax, an element-wise sigmoid output gate); a latent attention with queries
    through a latent of their own and an interleaved rotary on the shared key part, optionally reading
    an earlier layer's cache; a gated delta rule with channel-wise decay.  Feed-forward: dense, gated
    tanh-GELU, or none.  Untied head."""
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m = L["mixer"]
        rot = m.get("rot") or {}
        if L["type"] == "attention":
            mixer = GqaAttention(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), rot_layout="halves", mask="causal",
                values_are_keys=True, qk_bias=True, sink=True, out_gate=True, rot_scaling=_rot_scaling(rot))
            if mixer.vdim != mixer.dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim {mixer.vdim} must equal dim {mixer.dim}")
        elif L["type"] == "latent_attention":
            mixer = LatentAttention(
                heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                window=0, rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot.get("base", 10000.0)), scale=float(m["scale"]),
                kv_from=None if m.get("kv_from") is None else int(m["kv_from"]), q_rank=int(m["q_rank"]), rot_layout="interleaved",
                head_gate=False, rot_scaling=_rot_scaling(rot))
        elif L["type"] == "channel_delta":
            # the ranks of the decay and gate projections are sizes only the tensors give (0: taken from them)
            mixer = ChannelDelta(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                 conv=int(m["conv"]), rank_a=int(m.get("rank_a", 0)), rank_g=int(m.get("rank_g", 0)))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        f = L.get("mlp")
        if f is None:
            mlp = None
        elif f["kind"] == "dense":
            mlp = FeedForward("dense", int(f["ff"]), act="gelu_tanh_gated")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mixer, mlp))
    streams = int(cfg.get("streams") or 0)
    taps = int((cfg.get("canon") or {}).get("taps", 0))
    if streams < 0 or streams > 32:
        raise ValueError(f"streams {streams}: at most 32 residual streams")
    return LayeredSpec(name, int(cfg["width"]), int(cfg["vocab"]), float(cfg["norm"]["eps"]), tuple(layers), depth_mix=False,
                       block="prenorm", tied_head=False, norm_offset=1.0, streams=streams, canon_taps=taps, embed_norm=True)


ARCHITECTURES = {"Tivazen": _tivazen_from_config, "Nodutar": _nodutar_from_config, "Lugipel": _lugipel_from_config,
                 "Verelorn": _verelorn_from_config}


def spec_from_config(cfg: dict, name: str = "model", numerics: str = "hf"):
    """The spec class a config.json asks for: a layered design named by "architecture", else the
    Qwen decoder (HuggingFace keys)."""
    arch = cfg.get("architecture")
    if arch is not None:
        if arch not in ARCHITECTURES:
            raise ValueError(f"unknown architecture {arch!r} (known: {sorted(ARCHITECTURES)})")
        return ARCHITECTURES[arch](cfg, name)
    return ModelSpec.from_hf_config(cfg, name=name, numerics=numerics)


def with_tensor_sizes(spec, shapes: "dict[str, List[int]]"):
    """Sizes a config leaves to the checkpoint's tensors (the ranks of a ChannelDelta's decay and gate
    projections), filled in from a name -> shape table."""
    if not isinstance(spec, LayeredSpec):
        return spec
    layers = list(spec.layers)
    for i, L in enumerate(layers):
        m = L.mixer
        if isinstance(m, ChannelDelta) and (m.rank_a == 0 or m.rank_g == 0):
            a1, g1 = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.g1")
            if a1 is None or g1 is None:
                raise ValueError(f"layer {i}: tensors 'l{i}.mix.a1' / 'l{i}.mix.g1' are missing")
            layers[i] = LayerSpec(dataclasses.replace(m, rank_a=m.rank_a or int(a1[0]), rank_g=m.rank_g or int(g1[0])), L.mlp)
    return dataclasses.replace(spec, layers=tuple(layers))


def spec_from_dir(path: str, numerics: str = "hf"):
    import os
    with open(os.path.join(path, "config.json")) as f:
        spec = spec_from_config(json.load(f), name=os.path.basename(os.path.normpath(path)), numerics=numerics)
    st = os.path.join(path, "model.safetensors")
    if isinstance(spec, LayeredSpec) and os.path.exists(st) and any(
            isinstance(L.mixer, ChannelDelta) and 0 in (L.mixer.rank_a, L.mixer.rank_g) for L in spec.layers):
        import struct
        with open(st, "rb") as f:
            n = struct.unpack("<Q", f.read(8))[0]
            hdr = json.loads(f.read(n))
        spec = with_tensor_sizes(spec, {k: v["shape"] for k, v in hdr.items() if k != "__metadata__"})
    return spec
