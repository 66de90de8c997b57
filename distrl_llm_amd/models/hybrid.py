"""Layer-list ("hybrid") decoder models: every layer names its own mixer.

The dense families in ``model.py`` repeat one block; the models here are
described by a list of layers, each with a token mixer of some kind
(windowed latent attention, a minGRU recurrence, ...) and an optional
mixture-of-experts feed-forward. A design is a small table that maps its
``config.json`` onto these generic layer specs and its tensor names onto
the packed weights the engine's step function reads; the mechanisms
themselves (``ops/seqmix.py``) take every size and constant as a
parameter, so another design can reuse them in another order.

``Nibalix`` is the first design of this kind:

* residual stream in fp32; one offset-weight RMS norm per layer feeds both
  sublayers (parallel arrangement), ``x += m * (g1*mixer + g2*ff)`` with
  sigmoid gates read from the normed input;
* the mixer reads ``h + conv(h)``, a short causal depthwise convolution;
* mixers: latent attention (a low-rank latent plus one rotated key part
  shared by the heads is all that is cached; sliding window; a layer may
  read another layer's cache) and minGRU (gates depend on the current
  token only; fp32 state carried per sequence);
* feed-forward: top-k mixture of SiLU-gated experts, softmax over the
  chosen logits.

``Nedasun`` is the second:

* residual stream in fp32; sequential sublayers, each with an offset RMS
  norm before and after it (sandwich arrangement),
  ``x += norm_b(mixer(norm_a(x)))`` then the same around the feed-forward;
* mixers: grouped-query softmax attention over a paged K/V cache
  (interleaved-pair rotary on part of each head, tanh-capped scores, a
  learned per-head sink in the softmax denominator, the heads' weights
  mixed by a learned matrix, values blended with the first such layer's
  values) and the gated delta rule (short causal convolutions with SiLU on
  q/k/v, unit-norm q/k, per-head decay and write strength, fp32 matrix
  state per head and sequence, gated RMS norm on the read-out);
* feed-forward: a clamped GLU, dense or as a mixture of experts whose
  router takes a softmax over all outputs, chooses with an added
  correction, scales the unnormalised scores, may name identity experts
  and adds an always-on shared expert.

``Kakilorn`` is the third:

* residual stream in fp32, sublayers read it as it is and only their
  output is normed (post-norm arrangement, plain norm weights):
  ``x += norm(mixer(x))`` then ``x += norm(ff(x))``; the embedding is
  scaled and also serves, scaled again, as the output matrix;
* mixers: latent attention with low-rank queries, interleaved-pair rotary
  whose frequencies are rescaled for long contexts, a per-head sink in the
  softmax and a per-head sigmoid output gate; the gated delta rule with a
  decay per head *and key channel* (low-rank decay input, low-rank sigmoid
  output gate); and a parallel pair read from the same input: sigmoid
  attention (no softmax; RMS-normed q/k, a linear distance penalty per
  head, a sliding window that also keeps the first tokens) beside the
  per-head gated delta rule, summed with fixed scales;
* feed-forward: a dense SiLU-gated GLU.

``Legilix`` is the fourth:

* residual stream in fp32, pre-norm sublayers ``x += mixer(norm(x))`` then
  ``x += ff(norm(x))``; the norm is an RMS norm taken separately over equal
  consecutive groups of the width (plain weights); scaled embedding that
  also serves as the output matrix;
* mixers: two forms of grouped-query softmax attention with q/k/v biases
  under a sliding window (:class:`WindowAttentionSpec`): one with RMS-normed
  queries and keys, half-layout rotary on part of each head with rescaled
  frequencies, the heads' *scores* mixed by a learned matrix before the
  softmax and a window that keeps the first tokens; one without rotation,
  with a logarithmic distance bias per head and a per-head sigmoid output
  gate;
* feed-forward: a plain two-matrix MLP with tanh-GELU, or a mixture of
  SiLU-gated experts routed by sigmoid scores that are not renormalised and
  scale the expert's *input*.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn


# ------------------------------------------------------------------ specs

@dataclass(frozen=True)
class LatentAttentionSpec:
    heads: int
    dim: int            # unrotated q/k dims per head
    rot_dim: int        # rotated q/k dims per head (the key part is shared)
    vdim: int
    kv_rank: int
    scale: float
    rope_base: float
    rope_dims: int      # how many of the rot_dim entries are rotated
    window: int         # 0 = unbounded causal
    kv_from: Optional[int] = None   # layer whose cache this layer reads
    q_rank: int = 0     # > 0: queries go through a normed latent of this size
    rope_pairs: bool = False        # rotate entries (2i, 2i+1), else (i, i + dims/2)
    # long-context frequency rescaling: (factor, original length, fast turns,
    # slow turns), None = plain frequencies
    rope_scaling: Optional[tuple] = None
    sink: bool = False  # a learned per-head term in the softmax denominator
    out_gate: bool = False          # per-head sigmoid gate read from the mixer input

    kind = "latent_attention"

    @property
    def in_size(self) -> int:
        """Rows of the packed projection of the mixer input."""
        n = self.q_rank if self.q_rank else self.q_size
        if self.kv_from is None:
            n += self.cache_width
        return n + (self.heads if self.out_gate else 0)

    def rope_table(self):
        """(per-pair frequencies, factor on cos and sin) in double precision."""
        return rotary_frequencies(self.rope_dims, self.rope_base, self.rope_scaling)

    @property
    def q_size(self) -> int:
        return self.heads * (self.dim + self.rot_dim)

    @property
    def cache_width(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class MinGRUSpec:
    width: int
    kind = "mingru"

    @property
    def state_size(self) -> int:
        return self.width


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query softmax attention over paged K/V rows."""
    heads: int
    kv_heads: int
    dim: int            # q/k dims per head
    vdim: int
    scale: float
    softcap: float      # 0 = scores are not capped
    rope_base: float
    rope_dims: int      # leading dims of each head rotated as (2i, 2i+1) pairs
    v_first: Optional[int] = None   # layer whose fresh values are blended in
    v_mix: bool = False             # this layer takes part in value mixing

    kind = "sink_attention"

    @property
    def in_size(self) -> int:
        return self.q_size + self.cache_width

    @property
    def q_size(self) -> int:
        return self.heads * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def cache_width(self) -> int:      # one cache row = [k heads | v heads]
        return self.k_size + self.v_size


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta rule with short convolutions on q, k and v."""
    heads: int          # value heads (one state matrix each)
    kv_heads: int       # q/k heads, shared by heads // kv_heads value heads
    dim: int
    vdim: int
    taps: int
    # decay "head": one per head from a [H, D] projection; "channel": one per
    # head and key channel through a low-rank pair of projections
    decay: str = "head"
    decay_rank: int = 0
    # output gate: "silu" of a full projection, or "sigmoid" of a low-rank pair
    gate: str = "silu"
    gate_rank: int = 0

    kind = "delta_rule"

    @property
    def in_size(self) -> int:
        return self.conv_channels + (self.gate_rank if self.gate_rank else self.v_size)

    @property
    def ab_rows(self) -> int:           # fp32 rows: write strength | decay input
        return self.heads + (self.decay_rank if self.decay == "channel" else self.heads)

    @property
    def qk_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:    # q | k | v, convolved together
        return 2 * self.qk_size + self.v_size

    @property
    def state_size(self) -> int:
        return self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class SigmoidAttentionSpec:
    """Grouped-query attention whose weights are sigmoids of the scores (no
    normalisation over keys), with RMS-normed queries and keys, a linear
    distance penalty ``2^(-slope_exp (h+1) / H) * (i - j)`` per head, and a
    sliding window that also keeps the first ``keep_first`` tokens."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int         # 0 = unbounded causal
    keep_first: int
    slope_exp: float = 8.0

    kind = "sigmoid_attention"

    @property
    def q_size(self) -> int:
        return self.heads * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def in_size(self) -> int:
        return self.q_size + self.k_size + self.v_size

    @property
    def cache_width(self) -> int:      # one cache row = [k heads | v heads]
        return self.k_size + self.v_size

    def slopes(self):
        return [2.0 ** (-self.slope_exp * (h + 1) / self.heads)
                for h in range(self.heads)]


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Grouped-query softmax attention over paged [k | v] rows under a
    sliding window that may keep the first ``keep_first`` tokens. Options,
    each off by default: biases on q/k/v, RMS norm of every q and k head
    (plain shared weights), half-layout rotary (entry i pairs with
    i + dims/2) on the first ``rope_dims`` entries with optionally rescaled
    frequencies, mixing of the heads' scores by a learned [H, H] matrix
    before the softmax, a distance bias ``-r1_h ln(1 + r2_h (i - j))`` and a
    per-head sigmoid gate read from the mixer input."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0         # 0 = unbounded causal
    keep_first: int = 0
    qkv_bias: bool = False
    qk_norm: bool = False
    rope_dims: int = 0
    rope_base: float = 10000.0
    rope_scaling: Optional[tuple] = None
    score_mix: bool = False
    log_distance: bool = False
    out_gate: bool = False

    kind = "window_attention"

    @property
    def q_size(self) -> int:
        return self.heads * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def in_size(self) -> int:          # [q | k | v | gate]
        return (self.q_size + self.k_size + self.v_size
                + (self.heads if self.out_gate else 0))

    @property
    def cache_width(self) -> int:      # one cache row = [k heads | v heads]
        return self.k_size + self.v_size

    def rope_table(self):
        """(per-pair frequencies, factor on cos and sin) in double precision."""
        return rotary_frequencies(self.rope_dims, self.rope_base, self.rope_scaling)


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers that read the same input; the result is
    ``left_scale * left + right_scale * right``."""
    left: object
    right: object
    left_scale: float
    right_scale: float

    kind = "parallel"

    @property
    def in_size(self) -> int:
        return self.left.in_size + self.right.in_size


def mixer_units(spec: "HybridSpec"):
    """Every mixer that owns cache rows or state, with its key: the layer
    index, or (layer index, side) for the sides of a parallel pair."""
    for i, ls in enumerate(spec.layers):
        m = ls.mixer
        if isinstance(m, ParallelMixerSpec):
            yield (i, 0), m.left
            yield (i, 1), m.right
        else:
            yield i, m


def rotary_frequencies(dims: int, base: float, scaling: Optional[tuple] = None):
    """Per-pair rotary frequencies ``base^(-2i/dims)`` and the factor on cos
    and sin. With ``scaling = (factor, original, fast, slow)`` the pairs
    that turn fewer than ``slow`` times over ``original`` positions are
    slowed by ``factor``, those that turn more than ``fast`` times are kept,
    the ones between are blended linearly over the pair index, and cos/sin
    grow by ``0.1 ln(factor) + 1``."""
    half = dims // 2
    f = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    factor, original, fast, slow = (float(v) for v in scaling)

    def pair_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), dims - 1)
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


@dataclass(frozen=True)
class GluSpec:
    """Gated linear unit. ``act`` "capped": g = min(gate, limit),
    u = clamp(up, +-limit), y = g * sigmoid(1.702 g) * (u + 1); "silu":
    y = silu(gate) * up (limit unused)."""
    ff: int
    limit: float = 0.0
    act: str = "capped"


@dataclass(frozen=True)
class MlpSpec:
    """Plain two-matrix feed-forward ``down(act(up h))``; ``act``
    "gelu_tanh": 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""
    ff: int
    act: str = "gelu_tanh"


@dataclass(frozen=True)
class MoESpec:
    experts: int
    top: int
    ff: int
    # routing "chosen": softmax over the chosen logits; "all": softmax over
    # every router output, choice by score + correction, weight = score * scale;
    # "sigmoid": score = sigmoid(logit), the largest are chosen, weight = score
    routing: str = "chosen"
    # the weight multiplies the expert's input (expert(w h)) instead of its
    # output
    scale_input: bool = False
    identity: int = 0       # trailing router outputs that pass the input through
    scale: float = 1.0
    limit: float = 0.0      # 0: SiLU-gated experts; > 0: clamped GLU experts
    shared: Optional[GluSpec] = None


@dataclass(frozen=True)
class LayerSpec:
    mixer: object
    mlp: object         # MoESpec, GluSpec, MlpSpec or None


@dataclass(frozen=True)
class HybridSpec:
    name: str
    vocab_size: int
    width: int
    norm_eps: float
    residual_mult: float
    conv_taps: int
    layers: tuple = field(default_factory=tuple)
    # "parallel_gated": one norm feeds mixer and feed-forward, gated sum;
    # "sandwich": norm before and after each sublayer, one after the other;
    # "post_norm": sublayers read the residual, only their output is normed;
    # "pre_norm": x += sublayer(norm(x)), nothing else
    block: str = "parallel_gated"
    design: str = "nibalix"
    norm_offset: float = 1.0    # norm weights act as (offset + w)
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    tied_head: bool = False     # the embedding table is the output matrix
    # norms are taken separately over this many equal consecutive parts of
    # the width
    norm_groups: int = 1

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def nibalix_spec_from_config(cfg: dict, name: str = "nibalix") -> HybridSpec:
    """Map a Nibalix ``config.json`` onto the generic layer specs."""
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        if lc["type"] == "latent_attention":
            rot = mc.get("rot") or {}
            mixer = LatentAttentionSpec(
                heads=int(mc["heads"]), dim=int(mc["dim"]),
                rot_dim=int(mc["rot_dim"]), vdim=int(mc["vdim"]),
                kv_rank=int(mc["kv_rank"]),
                scale=float(mc["scale"] if mc.get("scale") is not None
                            else (int(mc["dim"]) + int(mc["rot_dim"])) ** -0.5),
                rope_base=float(rot.get("base") or 10000.0),
                rope_dims=int(rot["dims"] if rot.get("dims") is not None
                              else mc["rot_dim"]),
                window=int((mc.get("mask") or {}).get("size") or 0),
                kv_from=(int(mc["kv_from"]) if mc.get("kv_from") is not None
                         else None))
            if mixer.rope_dims > mixer.rot_dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and "
                                 f"<= rot_dim")
        elif lc["type"] == "mingru":
            mixer = MinGRUSpec(width=int(mc["width"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
        fc = lc.get("mlp")
        mlp = None
        if fc is not None:
            if fc.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown mlp kind {fc['kind']!r}")
            mlp = MoESpec(experts=int(fc["router"]["experts"]),
                          top=int(fc["router"]["top"]),
                          ff=int(fc["expert"]["ff"]))
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"layer {i}: top must be in [1, experts]")
        layers.append(LayerSpec(mixer, mlp))
    for i, ls in enumerate(layers):
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec) and m.kv_from is not None:
            src = layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
            if (not isinstance(src, LatentAttentionSpec)
                    or src.kv_from is not None
                    or src.cache_width != m.cache_width
                    or src.kv_rank != m.kv_rank):
                raise ValueError(f"layer {i}: kv_from must name an earlier "
                                 f"latent layer with a cache of its own and "
                                 f"equal kv_rank/rot_dim")
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]),
                      residual_mult=float(cfg["residual_mult"]),
                      conv_taps=int((cfg.get("canon") or {}).get("taps") or 0),
                      layers=tuple(layers))


def nibalix_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`nibalix_spec_from_config` (checkpoint saving)."""
    layers = []
    for ls in spec.layers:
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec):
            mc = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims}}
            if m.window:
                mc["mask"] = {"size": m.window}
            if m.kv_from is not None:
                mc["kv_from"] = m.kv_from
            typ = "latent_attention"
        else:
            mc, typ = {"width": m.width}, "mingru"
        fc = None
        if ls.mlp is not None:
            fc = {"kind": "moe", "expert": {"ff": ls.mlp.ff},
                  "router": {"experts": ls.mlp.experts, "top": ls.mlp.top}}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    out = {"architecture": "Nibalix", "layers": layers,
           "norm": {"eps": spec.norm_eps},
           "residual_mult": spec.residual_mult, "vocab": spec.vocab_size,
           "width": spec.width}
    if spec.conv_taps:
        out["canon"] = {"taps": spec.conv_taps}
    return out


# ---------------------------------------------------------------- weights

def _make_mixer_weights(mod, m, D, P, packed_input=True):
    """Create one mixer's packed parameters as attributes of ``mod``.
    ``packed_input`` False: the projection of the mixer input is owned by
    the caller (the sides of a parallel pair share one)."""
    f32 = torch.float32
    if packed_input:
        mod.in_w = P(m.in_size if hasattr(m, "in_size") else 3 * m.width, D)
    if isinstance(m, LatentAttentionSpec):
        if m.kv_from is None:
            mod.latent_norm_w = P(m.kv_rank, dt=f32)
        if m.q_rank:
            mod.q_norm_w = P(m.q_rank, dt=f32)
            mod.uq = P(m.q_size, m.q_rank)
        if m.sink:
            mod.sink = P(m.heads, dt=f32)
        mod.uk = P(m.heads, m.dim, m.kv_rank)
        mod.uv = P(m.heads, m.vdim, m.kv_rank)
        mod.out_w = P(D, m.heads * m.vdim)
    elif isinstance(m, SinkAttentionSpec):
        mod.talk = P(m.heads, m.heads, dt=f32)
        mod.sink = P(m.heads, dt=f32)
        mod.vmix = P(1, dt=f32)
        mod.out_w = P(D, m.heads * m.vdim)
    elif isinstance(m, SigmoidAttentionSpec):
        mod.q_norm_w, mod.k_norm_w = P(m.dim, dt=f32), P(m.dim, dt=f32)
        mod.pos_bias = P(m.heads, dt=f32)
        mod.out_w = P(D, m.heads * m.vdim)
    elif isinstance(m, WindowAttentionSpec):
        if m.qkv_bias:                  # added by the projection GEMM
            mod.in_b = P(m.in_size)
        if m.qk_norm:
            mod.q_norm_w, mod.k_norm_w = P(m.dim, dt=f32), P(m.dim, dt=f32)
        if m.score_mix:
            mod.talk = P(m.heads, m.heads, dt=f32)
        if m.log_distance:
            mod.dist_r1, mod.dist_r2 = P(m.heads, dt=f32), P(m.heads, dt=f32)
        mod.out_w = P(D, m.heads * m.vdim)
    elif isinstance(m, DeltaRuleSpec):
        mod.conv_w = P(m.conv_channels, m.taps, dt=f32)
        mod.ab_w = P(m.ab_rows, D, dt=f32)      # [write strength; decay input]
        mod.a_log = P(m.heads, dt=f32)
        if m.decay == "channel":
            mod.decay_up = P(m.heads * m.dim, m.decay_rank, dt=f32)
            mod.dt_bias = P(m.heads * m.dim, dt=f32)
        else:
            mod.dt_bias = P(m.heads, dt=f32)
        if m.gate_rank:
            mod.gate_up = P(m.v_size, m.gate_rank)
        mod.onorm_w = P(m.vdim, dt=f32)
        mod.out_w = P(D, m.v_size)
    else:
        mod.in_b = P(3 * m.width, dt=f32)
        mod.out_w = P(D, m.width)


class HybridLayer(nn.Module):
    """Packed inference weights of one layer.

    Projections that read the same input are stacked along the output
    axis so each input feeds one GEMM: ``in_w`` = [q; dkv] (latent),
    [z; x; g] (minGRU), [q; k; v] (sink attention) or [q; k; v; g] (delta
    rule); ``exp_gu``/``gu_w`` = [gate; up]. The block arrangement adds its
    own tensors: ``gate_w`` = [rg1; rg2] on the normed input (parallel
    gated), or the norms before/after each sublayer (sandwich)."""

    def __init__(self, spec: HybridSpec, ls: LayerSpec, dtype, device):
        super().__init__()
        D = spec.width

        def P(*shape, dt=dtype):
            return nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                requires_grad=False)

        f32 = torch.float32
        if spec.block == "post_norm":
            self.post_w = P(D, dt=f32)
            if ls.mlp is not None:
                self.ff_post_w = P(D, dt=f32)
        elif spec.block == "pre_norm":
            self.norm_w = P(D, dt=f32)
            if ls.mlp is not None:
                self.ff_norm_w = P(D, dt=f32)
        elif spec.block == "sandwich":
            self.norm_w = P(D, dt=f32)
            self.post_w = P(D, dt=f32)
            if ls.mlp is not None:
                self.ff_norm_w, self.ff_post_w = P(D, dt=f32), P(D, dt=f32)
        else:
            self.norm_w = P(D, dt=f32)
            if spec.conv_taps:  # 0: the mixer reads the normed input as it is
                self.conv_w = P(D, spec.conv_taps, dt=f32)
            n_gate = 2 * D if ls.mlp is not None else D
            self.gate_w, self.gate_b = P(n_gate, D), P(n_gate, dt=f32)
        m = ls.mixer
        if isinstance(m, ParallelMixerSpec):
            # both sides read one packed projection of the shared input
            self.in_w = P(m.in_size, D)
            self.left, self.right = nn.Module(), nn.Module()
            _make_mixer_weights(self.left, m.left, D, P, packed_input=False)
            _make_mixer_weights(self.right, m.right, D, P, packed_input=False)
        else:
            _make_mixer_weights(self, m, D, P)
        f = ls.mlp
        if isinstance(f, GluSpec):
            self.gu_w, self.down_w = P(2 * f.ff, D), P(D, f.ff)
        elif isinstance(f, MlpSpec):
            self.up_w, self.down_w = P(f.ff, D), P(D, f.ff)
        elif f is not None:
            n = f.experts + f.identity
            self.router_w = P(n, D, dt=f32)
            if f.routing != "sigmoid":
                self.router_b = P(n, dt=f32)
            if f.routing == "all":
                self.correction = P(n, dt=f32)
            self.exp_gu = P(f.experts, 2 * f.ff, D)
            self.exp_down = P(f.experts, D, f.ff)
            if f.shared is not None:
                self.shared_gu = P(2 * f.shared.ff, D)
                self.shared_down = P(D, f.shared.ff)


class HybridLM(nn.Module):
    """Inference weights of a layer-list model. ``dtype`` is the matrix
    dtype (bf16 or fp32); norm, conv, bias and router tensors stay fp32."""

    def __init__(self, spec: HybridSpec, dtype: torch.dtype = torch.bfloat16,
                 device=None):
        super().__init__()
        self.spec = spec
        self.dtype_ = dtype
        D = spec.width
        f32 = torch.float32

        def P(*shape, dt=dtype):
            return nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                requires_grad=False)

        self.embed = P(spec.vocab_size, D)
        if spec.design == "nibalix":
            self.embed_norm_w = P(D, dt=f32)
        self.final_norm_w = P(D, dt=f32)
        # a tied output matrix is the embedding parameter itself
        self.head = self.embed if spec.tied_head else P(spec.vocab_size, D)
        self.layers = nn.ModuleList(
            [HybridLayer(spec, ls, dtype, device) for ls in spec.layers])

    @property
    def device(self):
        return self.embed.device

    # ---- the design's tensor names <-> packed weights -------------------

    def _named_slices(self) -> Dict[str, tuple]:
        """{checkpoint tensor name: (packed parameter, row0, rows | None)}.
        ``rows`` None means the tensor fills the whole parameter; expert
        entries carry an index tuple instead of a row range."""
        if self.spec.design == "nedasun":
            return _nedasun_named_slices(self)
        if self.spec.design == "kakilorn":
            return _kakilorn_named_slices(self)
        if self.spec.design == "legilix":
            return _legilix_named_slices(self)
        out = {"embed": (self.embed, None), "embed.norm": (self.embed_norm_w, None),
               "final.norm": (self.final_norm_w, None), "head": (self.head, None)}
        D = self.spec.width
        for i, (ls, L) in enumerate(zip(self.spec.layers, self.layers)):
            p = f"l{i}."
            out[p + "norm1"] = (L.norm_w, None)
            if self.spec.conv_taps:
                out[p + "canon1"] = (L.conv_w, None)
            out[p + "rg1"], out[p + "rg1.b"] = (L.gate_w, (0, D)), (L.gate_b, (0, D))
            m = ls.mixer
            if isinstance(m, LatentAttentionSpec):
                out[p + "mix.q"] = (L.in_w, (0, m.q_size))
                if m.kv_from is None:
                    out[p + "mix.dkv"] = (L.in_w, (m.q_size, m.cache_width))
                    out[p + "mix.dkv.norm"] = (L.latent_norm_w, None)
                out[p + "mix.uk"] = (L.uk, "flat")
                out[p + "mix.uv"] = (L.uv, "flat")
            else:
                n = m.width
                for k, nm in enumerate(("z", "x", "g")):
                    out[p + "mix." + nm] = (L.in_w, (k * n, n))
                out[p + "mix.z.b"] = (L.in_b, (0, n))
                out[p + "mix.x.b"] = (L.in_b, (n, n))
            out[p + "mix.o"] = (L.out_w, None)
            if ls.mlp is not None:
                f = ls.mlp
                out[p + "rg2"], out[p + "rg2.b"] = (L.gate_w, (D, D)), (L.gate_b, (D, D))
                out[p + "mlp.router"] = (L.router_w, None)
                out[p + "mlp.router.b"] = (L.router_b, None)
                for e in range(f.experts):
                    out[f"{p}mlp.e{e}.gate"] = (L.exp_gu[e], (0, f.ff))
                    out[f"{p}mlp.e{e}.up"] = (L.exp_gu[e], (f.ff, f.ff))
                    out[f"{p}mlp.e{e}.down"] = (L.exp_down[e], None)
        return out

    @staticmethod
    def _view(param, where):
        if where is None:
            return param
        if where == "flat":
            return param.view(-1, param.shape[-1])
        r0, n = where
        return param[r0:r0 + n]

    @torch.no_grad()
    def load_tensors(self, tensors: Dict[str, torch.Tensor], strict=True) -> int:
        names = self._named_slices()
        for k, v in tensors.items():
            if k not in names:
                if strict:
                    raise ValueError(f"unexpected checkpoint tensor {k!r}")
                continue
            dst = self._view(*names[k])
            if v.dim() == 0 and dst.numel() == 1:
                v = v.reshape(dst.shape)
            if tuple(dst.shape) != tuple(v.shape):
                raise ValueError(f"shape mismatch for {k}: checkpoint "
                                 f"{tuple(v.shape)} vs model {tuple(dst.shape)}")
            dst.copy_(v.to(dst.dtype))
        missing = set(names) - set(tensors)
        if strict and missing:
            raise ValueError(f"checkpoint misses tensors: {sorted(missing)[:8]}")
        return len(names) - len(missing)

    def export_tensors(self, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
        scalars = _SCALAR_TENSORS.get(self.spec.design, ())
        out = {}
        for k, w in self._named_slices().items():
            t = self._view(*w).detach().to(dtype).contiguous().cpu()
            out[k] = t.reshape(()) if k.rsplit(".", 1)[-1] in scalars else t
        return out

    @torch.no_grad()
    def random_init(self, seed: int = 3407) -> "HybridLM":
        """Deterministic random weights (synthetic benches and tests)."""
        dev = self.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, (param, where) in sorted(self._named_slices().items()):
            dst = self._view(param, where)
            r = torch.randn(dst.shape, generator=g, dtype=torch.float32, device=dev)
            last = name.rsplit(".", 1)[-1]
            if name == "embed":
                pass
            elif last == "talk":
                r = torch.eye(dst.shape[0], device=dev) + 0.2 * r
            elif last == "vmix":
                r = 0.3 + 0.1 * r
            elif last in ("r1", "r2"):
                r = 0.5 + 0.1 * r.abs()
            elif last == "conv":
                r *= 0.5
            elif dst.dim() >= 2 and "canon" not in name:
                r *= 1.0 / math.sqrt(dst.shape[-1])
            elif (name.endswith("dkv.norm") or name.endswith("mix.norm")
                  or (self.spec.norm_offset == 0.0 and last in
                      ("norm", "norm1", "norm2"))):
                r = 1.0 + 0.1 * r
            else:
                r *= 0.1
            dst.copy_(r.to(dst.dtype))
        return self


# ------------------------------------------------------------ checkpoints

def load_nibalix_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "nibalix"
    model = HybridLM(nibalix_spec_from_config(cfg, name), dtype=dtype, device=device)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[nibalix] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    model.load_tensors({k: v for k, v in tensors.items() if k in known})
    return model


def save_nibalix_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(nibalix_config_from_spec(model.spec), f, indent=1)


# ---------------------------------------------------------------- Nedasun

_SCALAR_TENSORS = {"nedasun": ("vmix",)}   # stored with shape ()


def _glu_from_config(fc: dict) -> GluSpec:
    return GluSpec(ff=int(fc["ff"]), limit=float(fc["limit"]))


def nedasun_spec_from_config(cfg: dict, name: str = "nedasun") -> HybridSpec:
    """Map a Nedasun ``config.json`` onto the generic layer specs."""
    layers, v_first = [], None
    for i, lc in enumerate(cfg["layers"]):
        mc = lc["mixer"]
        heads, kvh = int(mc["heads"]), int(mc["kv_heads"])
        if kvh < 1 or heads % kvh:
            raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        if lc["type"] == "attention":
            rot = mc.get("rot") or {}
            mixes = bool(mc.get("v_mix"))
            mixer = SinkAttentionSpec(
                heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                vdim=int(mc["vdim"]), scale=float(mc["scale"]),
                softcap=float(mc.get("softcap") or 0.0),
                rope_base=float(rot.get("base") or 10000.0),
                rope_dims=int(rot.get("dims") or 0), v_mix=mixes,
                v_first=v_first if mixes else None)
            if mixer.rope_dims > mixer.dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and <= dim")
            if mixes and v_first is None:
                v_first = i
            elif mixes and ((layers[v_first].mixer.kv_heads, layers[v_first].mixer.vdim)
                            != (kvh, mixer.vdim)):
                raise ValueError(f"layer {i}: value mixing needs the first "
                                 f"mixing layer's kv_heads and vdim")
        elif lc["type"] == "delta":
            mixer = DeltaRuleSpec(heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                                  vdim=int(mc["vdim"]), taps=int(mc["conv"]))
            if mixer.taps < 1:
                raise ValueError(f"layer {i}: conv needs at least one tap")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {lc['type']!r}")
        fc = lc.get("mlp")
        mlp = None
        if fc is not None and fc.get("kind") == "dense":
            mlp = _glu_from_config(fc)
        elif fc is not None and fc.get("kind") == "moe":
            rc = fc["router"]
            mlp = MoESpec(experts=int(rc["experts"]), top=int(rc["top"]),
                          ff=int(fc["expert"]["ff"]), routing="all",
                          identity=int(rc.get("identity") or 0),
                          scale=float(rc.get("scale", 1.0)),
                          limit=float(fc["expert"]["limit"]),
                          shared=(_glu_from_config(fc["shared"])
                                  if fc.get("shared") else None))
            if not 1 <= mlp.top <= mlp.experts + mlp.identity:
                raise ValueError(f"layer {i}: top must be in [1, experts + identity]")
            if mlp.limit <= 0:
                raise ValueError(f"layer {i}: expert limit must be positive")
        elif fc is not None:
            raise ValueError(f"layer {i}: unknown mlp kind {fc.get('kind')!r}")
        layers.append(LayerSpec(mixer, mlp))
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]), residual_mult=1.0,
                      conv_taps=0, layers=tuple(layers), block="sandwich",
                      design="nedasun")


def nedasun_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`nedasun_spec_from_config` (checkpoint saving)."""
    layers = []
    for ls in spec.layers:
        m = ls.mixer
        if isinstance(m, SinkAttentionSpec):
            mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "scale": m.scale, "softcap": m.softcap,
                  "rot": {"base": m.rope_base, "dims": m.rope_dims},
                  "v_mix": m.v_mix}
            typ = "attention"
        else:
            mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                  "vdim": m.vdim, "conv": m.taps}
            typ = "delta"
        f, fc = ls.mlp, None
        if isinstance(f, GluSpec):
            fc = {"kind": "dense", "ff": f.ff, "limit": f.limit}
        elif f is not None:
            fc = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit},
                  "router": {"experts": f.experts, "identity": f.identity,
                             "scale": f.scale, "top": f.top},
                  "shared": ({"ff": f.shared.ff, "limit": f.shared.limit}
                             if f.shared is not None else None)}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    return {"architecture": "Nedasun", "layers": layers,
            "norm": {"eps": spec.norm_eps}, "vocab": spec.vocab_size,
            "width": spec.width}


def _nedasun_named_slices(model: "HybridLM") -> Dict[str, tuple]:
    out = {"embed": (model.embed, None), "final.norm": (model.final_norm_w, None),
           "head": (model.head, None)}

    def glu(pre, gu, down, ff):
        out[pre + "gate"], out[pre + "up"] = (gu, (0, ff)), (gu, (ff, ff))
        out[pre + "down"] = (down, None)

    for i, (ls, L) in enumerate(zip(model.spec.layers, model.layers)):
        p, m = f"l{i}.", ls.mixer
        out[p + "norm1"], out[p + "norm1b"] = (L.norm_w, None), (L.post_w, None)
        x = p + "mix."
        if isinstance(m, SinkAttentionSpec):
            out[x + "q"] = (L.in_w, (0, m.q_size))
            out[x + "k"] = (L.in_w, (m.q_size, m.k_size))
            out[x + "v"] = (L.in_w, (m.q_size + m.k_size, m.v_size))
            out[x + "vmix"], out[x + "talk"] = (L.vmix, None), (L.talk, None)
            out[x + "sink"] = (L.sink, None)
        else:
            n, nv = m.qk_size, m.v_size
            for nm, r0, rows in (("q", 0, n), ("k", n, n), ("v", 2 * n, nv)):
                out[x + nm] = (L.in_w, (r0, rows))
                out[x + nm + ".conv"] = (L.conv_w, (r0, rows))
            out[x + "g"] = (L.in_w, (2 * n + nv, nv))
            out[x + "b"] = (L.ab_w, (0, m.heads))
            out[x + "a"] = (L.ab_w, (m.heads, m.heads))
            out[x + "A_log"], out[x + "dt_bias"] = (L.a_log, None), (L.dt_bias, None)
            out[x + "norm"] = (L.onorm_w, None)
        out[x + "o"] = (L.out_w, None)
        f = ls.mlp
        if f is None:
            continue
        out[p + "norm2"], out[p + "norm2b"] = (L.ff_norm_w, None), (L.ff_post_w, None)
        x = p + "mlp."
        if isinstance(f, GluSpec):
            glu(x, L.gu_w, L.down_w, f.ff)
            continue
        out[x + "router"], out[x + "correction"] = (L.router_w, None), (L.correction, None)
        for e in range(f.experts):
            glu(f"{x}e{e}.", L.exp_gu[e], L.exp_down[e], f.ff)
        if f.shared is not None:
            glu(x + "shared.", L.shared_gu, L.shared_down, f.shared.ff)
    return out


def load_nedasun_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "nedasun"
    model = HybridLM(nedasun_spec_from_config(cfg, name), dtype=dtype, device=device)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[nedasun] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    # the blend factor is read only by mixing layers after the first one: a
    # checkpoint may leave it out elsewhere
    unused = {f"l{i}.mix.vmix" for i, ls in enumerate(model.spec.layers)
              if isinstance(ls.mixer, SinkAttentionSpec) and ls.mixer.v_first is None}
    have = {k: v for k, v in tensors.items() if k in known}
    missing = set(known) - set(have) - unused
    if missing:
        raise ValueError(f"checkpoint misses tensors: {sorted(missing)[:8]}")
    model.load_tensors(have, strict=False)
    return model


def save_nedasun_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(nedasun_config_from_spec(model.spec), f, indent=1)


# --------------------------------------------------------------- Kakilorn

def _delta_from_config(i, mc, channel: bool) -> DeltaRuleSpec:
    heads, kvh = int(mc["heads"]), int(mc["kv_heads"])
    if kvh < 1 or heads % kvh:
        raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
    if int(mc["conv"]) < 1:
        raise ValueError(f"layer {i}: conv needs at least one tap")
    return DeltaRuleSpec(heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                         vdim=int(mc["vdim"]), taps=int(mc["conv"]),
                         decay="channel" if channel else "head",
                         gate="sigmoid" if channel else "silu")


def kakilorn_spec_from_config(cfg: dict, name: str = "kakilorn",
                              shapes: Optional[dict] = None) -> HybridSpec:
    """Map a Kakilorn ``config.json`` onto the generic layer specs. The
    ranks of the low-rank decay and gate inputs are not in the config: they
    are the row counts of the checkpoint's ``a1``/``g1`` tensors
    (``shapes``: tensor name -> shape), or ``decay_rank``/``gate_rank``
    entries of the mixer's config when a checkpoint is written from a spec."""
    shapes = shapes or {}
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc, typ = lc["mixer"], lc["type"]
        if typ == "latent_attention":
            rot = mc.get("rot") or {}
            sc = rot.get("scaling")
            mixer = LatentAttentionSpec(
                heads=int(mc["heads"]), dim=int(mc["dim"]),
                rot_dim=int(mc["rot_dim"]), vdim=int(mc["vdim"]),
                kv_rank=int(mc["kv_rank"]), scale=float(mc["scale"]),
                rope_base=float(rot.get("base") or 10000.0),
                rope_dims=int(rot["dims"] if rot.get("dims") is not None
                              else mc["rot_dim"]),
                window=0, q_rank=int(mc["q_rank"]), rope_pairs=True,
                rope_scaling=(None if not sc else
                              (float(sc["factor"]), float(sc["original"]),
                               float(sc["fast"]), float(sc["slow"]))),
                sink=True, out_gate=True)
            if mixer.rope_dims > mixer.rot_dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and <= rot_dim")
            if mixer.q_rank < 1:
                raise ValueError(f"layer {i}: q_rank must be positive")
        elif typ == "channel_delta":
            d = _delta_from_config(i, mc, True)
            ra = shapes.get(f"l{i}.mix.a1", (mc.get("decay_rank"),))[0]
            rg = shapes.get(f"l{i}.mix.g1", (mc.get("gate_rank"),))[0]
            if not ra or not rg:
                raise ValueError(f"layer {i}: the ranks of the decay and gate "
                                 f"inputs are unknown")
            mixer = DeltaRuleSpec(**{**d.__dict__, "decay_rank": int(ra),
                                     "gate_rank": int(rg)})
        elif typ == "parallel":
            lm, rm = mc["left"], mc["right"]
            heads, kvh = int(lm["heads"]), int(lm["kv_heads"])
            if kvh < 1 or heads % kvh:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            mask = lm.get("mask") or {}
            left = SigmoidAttentionSpec(
                heads=heads, kv_heads=kvh, dim=int(lm["dim"]),
                vdim=int(lm["vdim"]), scale=float(lm["scale"]),
                window=int(mask.get("size") or 0),
                keep_first=int(mask.get("keep_first") or 0))
            mixer = ParallelMixerSpec(left, _delta_from_config(i, rm, False),
                                      float(mc["left_scale"]),
                                      float(mc["right_scale"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {typ!r}")
        fc, mlp = lc.get("mlp"), None
        if fc is not None:
            if fc.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown mlp kind {fc.get('kind')!r}")
            mlp = GluSpec(ff=int(fc["ff"]), act="silu")
        layers.append(LayerSpec(mixer, mlp))
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]), residual_mult=1.0,
                      conv_taps=0, layers=tuple(layers), block="post_norm",
                      design="kakilorn", norm_offset=0.0,
                      embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                      logit_scale=float(cfg.get("logit_scale", 1.0)),
                      tied_head=True)


def kakilorn_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`kakilorn_spec_from_config` (checkpoint saving)."""
    def delta(m):
        return {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                "vdim": m.vdim, "conv": m.taps}

    layers = []
    for ls in spec.layers:
        m = ls.mixer
        if isinstance(m, LatentAttentionSpec):
            rot = {"base": m.rope_base, "dims": m.rope_dims}
            if m.rope_scaling:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"),
                                          m.rope_scaling))
            mc = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim,
                  "vdim": m.vdim, "kv_rank": m.kv_rank, "q_rank": m.q_rank,
                  "scale": m.scale, "rot": rot}
            typ = "latent_attention"
        elif isinstance(m, DeltaRuleSpec):
            mc, typ = delta(m), "channel_delta"
        else:
            a = m.left
            left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim,
                    "vdim": a.vdim, "scale": a.scale}
            if a.window:
                left["mask"] = {"size": a.window, "keep_first": a.keep_first}
            mc = {"left": left, "right": delta(m.right),
                  "left_scale": m.left_scale, "right_scale": m.right_scale}
            typ = "parallel"
        fc = None if ls.mlp is None else {"kind": "dense", "ff": ls.mlp.ff}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    return {"architecture": "Kakilorn", "embedding": {"scale": spec.embed_scale},
            "layers": layers, "logit_scale": spec.logit_scale,
            "norm": {"eps": spec.norm_eps}, "vocab": spec.vocab_size,
            "width": spec.width}


def _kakilorn_named_slices(model: "HybridLM") -> Dict[str, tuple]:
    out = {"embed": (model.embed, None), "final.norm": (model.final_norm_w, None)}

    def delta(x, m, W, in_w, r0):
        """Names of a delta-rule mixer whose packed input rows start at r0."""
        n, nv = m.qk_size, m.v_size
        for nm, a, rows in (("q", 0, n), ("k", n, n), ("v", 2 * n, nv)):
            out[x + nm] = (in_w, (r0 + a, rows))
            out[x + nm + ".conv"] = (W.conv_w, (a, rows))
        c = r0 + m.conv_channels
        out[x + "b"] = (W.ab_w, (0, m.heads))
        if m.decay == "channel":
            out[x + "a1"] = (W.ab_w, (m.heads, m.decay_rank))
            out[x + "a2"] = (W.decay_up, None)
        else:
            out[x + "a"] = (W.ab_w, (m.heads, m.heads))
        if m.gate_rank:
            out[x + "g1"] = (in_w, (c, m.gate_rank))
            out[x + "g2"] = (W.gate_up, None)
        else:
            out[x + "g"] = (in_w, (c, nv))
        out[x + "A_log"], out[x + "dt_bias"] = (W.a_log, None), (W.dt_bias, None)
        out[x + "norm"], out[x + "o"] = (W.onorm_w, None), (W.out_w, None)

    for i, (ls, L) in enumerate(zip(model.spec.layers, model.layers)):
        p, m = f"l{i}.", ls.mixer
        x = p + "mix."
        out[p + "norm1"] = (L.post_w, None)
        if isinstance(m, LatentAttentionSpec):
            w = m.cache_width
            out[x + "dq"] = (L.in_w, (0, m.q_rank))
            out[x + "dkv"] = (L.in_w, (m.q_rank, w))
            out[x + "g"] = (L.in_w, (m.q_rank + w, m.heads))
            out[x + "dq.norm"], out[x + "uq"] = (L.q_norm_w, None), (L.uq, None)
            out[x + "dkv.norm"] = (L.latent_norm_w, None)
            out[x + "uk"], out[x + "uv"] = (L.uk, "flat"), (L.uv, "flat")
            out[x + "sink"], out[x + "o"] = (L.sink, None), (L.out_w, None)
        elif isinstance(m, DeltaRuleSpec):
            delta(x, m, L, L.in_w, 0)
        else:
            a, W = m.left, L.left
            y = x + "left."
            out[y + "q"] = (L.in_w, (0, a.q_size))
            out[y + "k"] = (L.in_w, (a.q_size, a.k_size))
            out[y + "v"] = (L.in_w, (a.q_size + a.k_size, a.v_size))
            out[y + "q.norm"], out[y + "k.norm"] = (W.q_norm_w, None), (W.k_norm_w, None)
            out[y + "pb"], out[y + "o"] = (W.pos_bias, None), (W.out_w, None)
            delta(x + "right.", m.right, L.right, L.in_w, a.in_size)
        if ls.mlp is not None:
            f = ls.mlp
            out[p + "norm2"] = (L.ff_post_w, None)
            out[p + "mlp.gate"] = (L.gu_w, (0, f.ff))
            out[p + "mlp.up"] = (L.gu_w, (f.ff, f.ff))
            out[p + "mlp.down"] = (L.down_w, None)
    return out


def _safetensors_shapes(path: str) -> dict:
    """Tensor name -> shape from a safetensors file's header."""
    import struct
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in head.items() if k != "__metadata__"}


def load_kakilorn_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "kakilorn"
    file = os.path.join(path, "model.safetensors")
    spec = kakilorn_spec_from_config(cfg, name, _safetensors_shapes(file))
    model = HybridLM(spec, dtype=dtype, device=device)
    tensors = load_file(file)
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[kakilorn] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    model.load_tensors({k: v for k, v in tensors.items() if k in known})
    return model


def save_kakilorn_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(kakilorn_config_from_spec(model.spec), f, indent=1)


# ---------------------------------------------------------------- Legilix

def legilix_spec_from_config(cfg: dict, name: str = "legilix") -> HybridSpec:
    """Map a Legilix ``config.json`` onto the generic layer specs."""
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        mc, typ = lc["mixer"], lc["type"]
        heads, kvh = int(mc["heads"]), int(mc["kv_heads"])
        if kvh < 1 or heads % kvh:
            raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        mask = mc.get("mask") or {}
        common = dict(heads=heads, kv_heads=kvh, dim=int(mc["dim"]),
                      vdim=int(mc["vdim"]), scale=float(mc["scale"]),
                      window=int(mask.get("size") or 0), qkv_bias=True)
        if typ == "attention":
            rot = mc.get("rot") or {}
            sc = rot.get("scaling")
            mixer = WindowAttentionSpec(
                **common, keep_first=int(mask.get("keep_first") or 0),
                qk_norm=True, rope_dims=int(rot.get("dims") or 0),
                rope_base=float(rot.get("base") or 10000.0),
                rope_scaling=(None if not sc else
                              (float(sc["factor"]), float(sc["original"]),
                               float(sc["fast"]), float(sc["slow"]))),
                score_mix=True)
            if mixer.rope_dims > mixer.dim or mixer.rope_dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and <= dim")
        elif typ == "attention_2":
            mixer = WindowAttentionSpec(**common, log_distance=True, out_gate=True)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {typ!r}")
        fc, mlp = lc.get("mlp"), None
        if fc is not None and fc.get("kind") == "dense":
            mlp = MlpSpec(ff=int(fc["ff"]))
        elif fc is not None and fc.get("kind") == "moe":
            rc = fc["router"]
            mlp = MoESpec(experts=int(rc["experts"]), top=int(rc["top"]),
                          ff=int(fc["expert"]["ff"]), routing="sigmoid",
                          scale_input=True)
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"layer {i}: top must be in [1, experts]")
        elif fc is not None:
            raise ValueError(f"layer {i}: unknown mlp kind {fc.get('kind')!r}")
        layers.append(LayerSpec(mixer, mlp))
    groups = int((cfg["norm"].get("groups")) or 1)
    if groups < 1 or int(cfg["width"]) % groups:
        raise ValueError("norm.groups must divide the width")
    return HybridSpec(name=name, vocab_size=int(cfg["vocab"]),
                      width=int(cfg["width"]),
                      norm_eps=float(cfg["norm"]["eps"]), residual_mult=1.0,
                      conv_taps=0, layers=tuple(layers), block="pre_norm",
                      design="legilix", norm_offset=0.0,
                      embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                      logit_scale=float(cfg.get("logit_scale", 1.0)),
                      tied_head=True, norm_groups=groups)


def legilix_config_from_spec(spec: HybridSpec) -> dict:
    """Inverse of :func:`legilix_spec_from_config` (checkpoint saving)."""
    layers = []
    for ls in spec.layers:
        m = ls.mixer
        mc = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
              "vdim": m.vdim, "scale": m.scale}
        if m.score_mix:
            typ = "attention"
            if m.window:
                mc["mask"] = {"size": m.window, "keep_first": m.keep_first}
            rot = {"base": m.rope_base, "dims": m.rope_dims}
            if m.rope_scaling:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"),
                                          m.rope_scaling))
            mc["rot"] = rot
        else:
            typ = "attention_2"
            if m.window:
                mc["mask"] = {"size": m.window}
        f, fc = ls.mlp, None
        if isinstance(f, MlpSpec):
            fc = {"kind": "dense", "ff": f.ff}
        elif f is not None:
            fc = {"kind": "moe", "expert": {"ff": f.ff},
                  "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": typ, "mixer": mc, "mlp": fc})
    return {"architecture": "Legilix", "embedding": {"scale": spec.embed_scale},
            "layers": layers, "logit_scale": spec.logit_scale,
            "norm": {"eps": spec.norm_eps, "groups": spec.norm_groups},
            "vocab": spec.vocab_size, "width": spec.width}


def _legilix_named_slices(model: "HybridLM") -> Dict[str, tuple]:
    out = {"embed": (model.embed, None), "final.norm": (model.final_norm_w, None)}
    for i, (ls, L) in enumerate(zip(model.spec.layers, model.layers)):
        p, m = f"l{i}.", ls.mixer
        x = p + "mix."
        out[p + "norm1"] = (L.norm_w, None)
        r0 = 0
        for nm, rows in (("q", m.q_size), ("k", m.k_size), ("v", m.v_size)):
            out[x + nm] = (L.in_w, (r0, rows))
            out[x + nm + ".b"] = (L.in_b, (r0, rows))
            r0 += rows
        if m.out_gate:                  # its rows of the packed bias stay zero
            out[x + "g"] = (L.in_w, (r0, m.heads))
        if m.qk_norm:
            out[x + "q.norm"], out[x + "k.norm"] = (L.q_norm_w, None), (L.k_norm_w, None)
        if m.score_mix:
            out[x + "talk"] = (L.talk, None)
        if m.log_distance:
            out[x + "r1"], out[x + "r2"] = (L.dist_r1, None), (L.dist_r2, None)
        out[x + "o"] = (L.out_w, None)
        f = ls.mlp
        if f is None:
            continue
        out[p + "norm2"] = (L.ff_norm_w, None)
        x = p + "mlp."
        if isinstance(f, MlpSpec):
            out[x + "up"], out[x + "down"] = (L.up_w, None), (L.down_w, None)
            continue
        out[x + "router"] = (L.router_w, None)
        for e in range(f.experts):
            out[f"{x}e{e}.gate"] = (L.exp_gu[e], (0, f.ff))
            out[f"{x}e{e}.up"] = (L.exp_gu[e], (f.ff, f.ff))
            out[f"{x}e{e}.down"] = (L.exp_down[e], None)
    return out


def load_legilix_checkpoint(path: str, dtype=torch.bfloat16, device=None) -> HybridLM:
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "legilix"
    model = HybridLM(legilix_spec_from_config(cfg, name), dtype=dtype, device=device)
    tensors = load_file(os.path.join(path, "model.safetensors"))
    known = model._named_slices()
    extra = sorted(k for k in tensors if k not in known)
    if extra:
        import sys
        sys.stderr.write(f"[legilix] ignoring {len(extra)} tensors the design "
                         f"does not name: {extra[:4]}\n")
    model.load_tensors({k: v for k, v in tensors.items() if k in known})
    return model


def save_legilix_checkpoint(model: HybridLM, path: str) -> None:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file(model.export_tensors(), os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(legilix_config_from_spec(model.spec), f, indent=1)
