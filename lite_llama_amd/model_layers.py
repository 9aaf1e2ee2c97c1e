"""Layered decoder models: a stack described layer by layer in ``config.json`` -- each layer names its sequence mixer, the
mixer's sizes and its feed-forward --, optionally with a span of layers that runs several times in a row with the same
weights.  Where model.py fixes ONE llama-shaped layer and a static geometry table, this file builds the stack from the
description, out of mixers that take a ragged step (executor/ragged.py) and keep their own kind of state in the
:class:`PagedStateCache`:

  * :class:`SinkAttention`     softmax attention, separate key / value widths, per-head q / k RMS norm, a position temperature
                               on the queries instead of a rotation, a learned sink in the denominator (kernels/attention.py)
  * :class:`GatedLinearMixer`  HGRN2: linear attention whose forget gate, bounded from below, also decides what is written
                               (kernels/recurrent.py)
  * :class:`DenseMLP`          ``down(act(up h))`` with the xIELU activation (kernels/activations.py)
  * :class:`LatentAttention`   attention over a shared low-rank latent with a rotated key part common to all heads, run in the
                               absorbed form (one key/value head over the cached latent rows), optionally with a query latent,
                               a sliding window and an output gate (kernels/attention.py)
  * :class:`MinGRU`            a per-channel gated recurrence whose gates read the current token only (kernels/recurrent.py)
  * :class:`GatedMLP`          ``down(act(gate h) * up h)`` (silu or tanh-gelu)
  * :class:`SparseMoE`         sigmoid router over expert groups, grouped expert products, a shared expert with a per-token
                               scale (kernels/fused_moe.py)
  * :class:`ConvRotaryAttention`  biased q / k / v behind a short causal convolution over time, a rotation of entry pairs, unit
                               RMS norm of q / k heads, a sliding window that also keeps a sequence's first keys, a sink of score
                               0 in the denominator, values blended with those of the first such layer (kernels/attention.py)
  * :class:`ChosenSoftmaxMoE`  the largest router logits choose the experts, their weights are the softmax over the chosen
                               logits alone (kernels/fused_moe.py)
  * :class:`WindowAttentionSSD`  two mixers side by side on one input: windowed softmax attention with whole-row q / k norms
                               and a rotation of (i, i + dims / 2) pairs, and a state-space mixer (short convolution, scalar
                               decay per head and token, gated grouped norm); one input and one output projection for both
  * :class:`DecayLinearAttention`  linear attention with a fixed decay per head over silu features (kernels/recurrent.py)
  * :class:`GatedLinearAttention`  linear attention with a decay per key entry from a low-rank projection
  * :class:`BiasedGatedMLP`    ``down(silu(gate h + b) * (up h + b)) + b``
  * :class:`CorrectedSoftmaxMoE`  softmax scores over all router outputs, experts chosen by score + correction and weighted by
                               the score alone, clamped expert activations, router outputs that stand for "the input itself"

The residual stream is fp32 throughout; every layer's residual add is fused into the norm that follows it
(kernels/norm_act.py::add_rmsnorm_shift, which also applies the token shift in front of a mixer; or
kernels/norm_act.py::gated_group_norm for layers that wrap each sublayer in two grouped norms and gate its result).
Projections run through the framework's linear layers (library GEMM for unquantised weights), with everything that reads one
input fused into one launch at load time.  Families: Rakevik (``"architecture": "Rakevik"``: :class:`MixerLayer`),
Rukedra (:class:`SandwichLayer`), Fekanex (:class:`ParallelLayer`: one norm per layer, mixer and feed-forward read its
output side by side, and -- with a dense feed-forward -- share ONE input projection and ONE output projection) and Nivotar
(:class:`PostNormLayer`: sublayers read the residual stream itself, the norm sits on each sublayer's result).
"""

from __future__ import annotations

import math
from collections.abc import Mapping
import dataclasses
from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from .distributed.parallel_state import get_tp_world_size
from .kernels.activations import xielu
from .kernels.attention import (conv_rope_cache, latent_kv_prep, qk_norm_cache, ragged_attention, rotate_pairs, rotation_table,
                                rownorm_rope_cache)
from .kernels.fused_moe import group_router, sparse_glu_experts
from .kernels.norm_act import (GatedUpdate, SummedUpdate, add_rmsnorm_shift, cast_pair, embed_pair, gated_group_norm, glu_act,
                               residual_set, softcap_)
from .kernels.recurrent import conv_act, gated_linear_scan, gated_out_norm, linear_scan, mingru_scan
from .linear import ReplicatedLinear


# ------------------------------------------------------------------------------------- #
# description
# ------------------------------------------------------------------------------------- #
@dataclass(frozen=True)
class RotarySpec:
    """Rotation of entry pairs (2i, 2i + 1) of the first ``dims`` entries by ``position * f_i``, ``f_i = base^(-2i / dims)``;
    with ``factor`` the frequencies are rescaled between a fast and a slow end (YaRN)."""
    dims: int
    base: float
    factor: float = 0.0         # 0: no scaling
    original: float = 0.0       # positions the unscaled frequencies were made for
    fast: float = 0.0           # turns over `original` positions above which a pair keeps its frequency
    slow: float = 0.0           # ... and below which it is divided by `factor`

    def table(self) -> tuple[list[float], float]:
        """``(frequency per pair, amplitude of cos / sin)``."""
        half = self.dims // 2
        f = [self.base ** (-2.0 * i / self.dims) for i in range(half)]
        if not self.factor:
            return f, 1.0

        def pair_of(turns: float) -> float:   # the (fractional) pair that makes `turns` turns over `original` positions
            return self.dims * math.log(self.original / (2 * math.pi * turns)) / (2 * math.log(self.base))

        lo = max(math.floor(pair_of(self.fast)), 0)
        hi = min(math.ceil(pair_of(self.slow)), self.dims - 1)
        out = []
        for i, fi in enumerate(f):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            out.append(fi / self.factor * ramp + fi * (1.0 - ramp))
        return out, 0.1 * math.log(self.factor) + 1.0

    @staticmethod
    def from_config(rot: Mapping) -> "RotarySpec":
        sc = rot.get("scaling")
        if not sc:
            return RotarySpec(int(rot["dims"]), float(rot["base"]))
        return RotarySpec(int(rot["dims"]), float(rot["base"]), float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                          float(sc["slow"]))


@dataclass(frozen=True)
class StateSpaceSpec:
    """The state-space half of a two-branch mixer: ``heads`` heads of ``vdim`` channels over a state of ``state`` entries,
    keys / queries shared by the heads of each of ``groups`` groups, a causal convolution of ``conv_taps`` taps in front, the
    gated read-out normed in ``norm_groups`` equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv_taps: int
    norm_groups: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass(frozen=True)
class MixerSpec:
    kind: str                   # "attention" | "hgrn2" | "latent_attention" | "mingru" | "conv_attention" | "attention_ssd" | "decay_linear" | "gla"
    heads: int = 1
    dim: int = 0                # per-head query / key width (latent attention: the unrotated part)
    vdim: int = 0               # per-head value width
    kv_heads: int = 0           # attention only
    scale: float = 1.0          # attention kinds
    temp_coef: float = 0.0      # attention only: q *= 1 + temp_coef ln(floor((p + 1) / temp_every) + 1)
    temp_every: int = 1
    rot_dim: int = 0            # latent attention: rotated query / key entries per head (the key's are shared by all heads)
    kv_rank: int = 0            # latent attention: width of the cached key/value latent
    q_rank: int = 0             # latent attention: width of the query latent (0: queries are projected directly)
    window: int = 0             # latent / conv attention: 0 = causal, else the last `window` positions are seen
    keep_first: int = 0         # conv attention: with a window, the sequence's first positions that stay visible
    bias: bool = False          # conv attention: q / k / v projections carry a bias
    conv_taps: int = 0          # conv attention: taps of the causal convolution over time behind the projections (0: none)
    unit_norm: bool = False     # conv attention: q / k heads divided by their root mean square (no weight) after the rotation
    unit_sink: bool = False     # conv attention: a key of score 0 without a value in every softmax denominator
    value_mix: bool = False     # conv attention: values blended with those of the first layer that says so
    out_gate: bool = False      # latent attention: heads times sigmoid(W_g h) before the output projection
    rotary: RotarySpec | None = None
    width: int = 0              # mingru: channels of the recurrence
    ssd: StateSpaceSpec | None = None           # attention_ssd: the state-space branch beside the attention
    branch_scales: tuple = (1.0, 1.0)           # attention_ssd: result = scales[0] * attention + scales[1] * state-space
    decay: tuple = ()           # decay_linear: the fixed decay of every head
    tau: float = 1.0            # gla: decay = sigmoid(.)^(1 / tau)
    decay_rank: int = 0         # gla: width of the low-rank projection in front of the decay logits


@dataclass(frozen=True)
class MlpSpec:
    kind: str = "dense"         # "dense" | "moe"
    ff: int = 0                 # dense: hidden width; moe: hidden width of one expert
    act: str = "xielu"          # dense: "xielu" (up / down) | "gelu_tanh" | "clamped" | "silu" (gate / up / down)
    limit: float = 0.0          # "clamped": gate <= limit, |up| <= limit
    scoring: str = "sigmoid"    # moe: "sigmoid" (scores over groups) | "softmax_chosen" (largest logits, softmax over them)
                                # | "softmax_all" (softmax over all outputs, chosen by score + correction)
    identity: int = 0           # moe, "softmax_all": router outputs beyond `experts` that stand for the input itself
    bias: bool = False          # dense: every projection carries a bias
    experts: int = 0
    top: int = 0
    group_count: int = 1
    group_keep: int = 1
    route_scale: float = 1.0
    shared_ff: int = 0          # 0: no shared expert


@dataclass(frozen=True)
class LayerSpec:
    mixer: MixerSpec
    ff: int = 0                 # 0: the layer has no feed-forward sublayer
    mlp_kind: str = "dense"
    mlp: MlpSpec | None = None
    weights_of: int | None = None   # the layer whose parameters this one uses (its cache / state stays its own)


@dataclass(frozen=True)
class LayeredGeometry:
    name: str
    vocab_size: int
    width: int
    eps: float
    layers: tuple[LayerSpec, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    token_shift: bool = True
    sandwich: bool = False      # every sublayer between two norms, its result gated by sigmoid(W_r h + b_r)
    norm_groups: int = 1        # norms are taken over this many equal consecutive parts of the row
    logit_softcap: float = 0.0  # logits <- cap tanh(logits / cap)
    parallel: bool = False      # one norm per layer; mixer and feed-forward both read it, their results are added together
    embed_scale: float = 1.0    # input = embedding row times this
    pair_buckets: int = 0       # > 0: plus row hash(previous token, token) of a [buckets + 1, width] table (last row: no previous)
    pair_mul_prev: int = 0      # hash = (previous * mul_prev + token * mul_cur) mod buckets
    pair_mul_cur: int = 0
    logit_scale: float = 1.0    # logits = head(norm(x)) times this
    tied_head: bool = False     # the output head is the embedding table
    post_norm: bool = False     # sublayers read the residual stream itself; each sublayer's RESULT is normed, then added
    extra: dict = field(default_factory=dict, compare=False)

    @property
    def looped(self) -> bool:
        return self.loop_stop > self.loop_start

    def run_order(self) -> list[tuple[int, int, bool]]:
        """``(layer index, pass number, first layer of a pass)`` per layer run."""
        n = len(self.layers)
        if not self.looped:
            return [(i, 0, False) for i in range(n)]
        order = [(i, 0, False) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            order += [(i, t, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return order + [(i, 0, False) for i in range(self.loop_stop, n)]

    @staticmethod
    def from_config(config: Mapping, name: str = "rakevik", shapes: Mapping | None = None) -> "LayeredGeometry":
        """``shapes``: ``{tensor name: shape}`` of the checkpoint, for sizes that only a tensor's shape gives."""
        if name == "nivotar":
            return _nivotar_geometry(config, name, shapes or {})
        if name == "rukedra":
            return _rukedra_geometry(config, name)
        if name == "fekanex":
            return _fekanex_geometry(config, name)
        layers = []
        for entry in config["layers"]:
            m, kind = entry["mixer"], entry["type"]
            if kind == "attention":
                temp = m.get("q_temp") or {}
                spec = MixerSpec("attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                 kv_heads=int(m.get("kv_heads") or m["heads"]), scale=float(m["scale"]),
                                 temp_coef=float(temp.get("coef", 0.0)), temp_every=int(temp.get("every", 1)))
                if spec.heads % spec.kv_heads:
                    raise ValueError(f"{spec.heads} query heads do not divide over {spec.kv_heads} key/value heads")
            elif kind == "hgrn2":
                spec = MixerSpec("hgrn2", int(m["heads"]), int(m["dim"]), int(m["vdim"]))
            else:
                raise ValueError(f"unsupported mixer type {kind!r}; supported: attention, hgrn2")
            mlp = entry.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}; supported: dense")
            layers.append(LayerSpec(spec, ff=int(mlp["ff"]) if mlp is not None else 0))
        loop = config.get("loop") or {}
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if stop > start and not (0 <= start < stop <= len(layers) and times >= 1):
            raise ValueError(f"loop {start}..{stop} x {times} does not fit {len(layers)} layers")
        return LayeredGeometry(name=name, vocab_size=int(config["vocab"]), width=int(config["width"]),
                               eps=float(config["norm"]["eps"]), layers=tuple(layers), loop_start=start, loop_stop=stop,
                               loop_times=times if stop > start else 1)


def _rukedra_geometry(config: Mapping, name: str) -> LayeredGeometry:
    """Rukedra: latent attention (two variants) and minGRU mixers, dense (tanh-gelu) and mixture-of-experts feed-forwards,
    grouped norms before and after every sublayer, gated residual branches, layers that borrow another layer's weights."""
    layers = []
    for index, entry in enumerate(config["layers"]):
        m, kind = entry["mixer"], entry["type"]
        if kind in ("latent_attention", "latent_attention_2"):
            first = kind == "latent_attention"
            rot = RotarySpec.from_config(m["rot"])
            spec = MixerSpec("latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                             scale=float(m["scale"]), rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]),
                             q_rank=int(m["q_rank"]) if first else 0, window=int((m.get("mask") or {}).get("size", 0)) if first else 0,
                             out_gate=first, rotary=rot)
            if rot.dims > spec.rot_dim or rot.dims % 2:
                raise ValueError(f"layer {index}: {rot.dims} rotated entries do not fit a rotated part of {spec.rot_dim}")
        elif kind == "mingru":
            spec = MixerSpec("mingru", width=int(m["width"]))
        else:
            raise ValueError(f"unsupported mixer type {kind!r}; supported: latent_attention, latent_attention_2, mingru")
        mlp = entry.get("mlp")
        if mlp is None:
            mspec = None
        elif mlp.get("kind", "dense") == "dense":
            mspec = MlpSpec("dense", ff=int(mlp["ff"]), act="gelu_tanh")
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            groups = r.get("groups") or {}
            mspec = MlpSpec("moe", ff=int(mlp["expert"]["ff"]), act="silu", experts=int(r["experts"]), top=int(r["top"]),
                            group_count=int(groups.get("count", 1)), group_keep=int(groups.get("keep", 1)),
                            route_scale=float(r.get("scale", 1.0)), shared_ff=int((mlp.get("shared") or {}).get("ff", 0)))
            if mspec.experts % mspec.group_count or mspec.group_keep * (mspec.experts // mspec.group_count) < mspec.top:
                raise ValueError(f"layer {index}: {mspec.top} of {mspec.experts} experts cannot be chosen from "
                                 f"{mspec.group_keep} of {mspec.group_count} groups")
        else:
            raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}; supported: dense, moe")
        owner = entry.get("weights_of")
        if owner is not None and not (0 <= int(owner) < len(config["layers"]) and int(owner) != index
                                      and config["layers"][int(owner)].get("weights_of") is None):
            raise ValueError(f"layer {index} borrows the weights of layer {owner}, which is not another layer with weights of its own")
        layers.append(LayerSpec(spec, ff=mspec.ff if mspec else 0, mlp_kind=mspec.kind if mspec else "dense", mlp=mspec,
                                weights_of=None if owner is None else int(owner)))
    norm = config["norm"]
    groups = int(norm.get("groups", 1))
    if int(config["width"]) % groups:
        raise ValueError(f"{groups} norm groups do not divide the width {config['width']}")
    return LayeredGeometry(name=name, vocab_size=int(config["vocab"]), width=int(config["width"]), eps=float(norm["eps"]),
                           layers=tuple(layers), token_shift=False, sandwich=True, norm_groups=groups,
                           logit_softcap=float(config.get("logit_softcap") or 0.0))


def _fekanex_geometry(config: Mapping, name: str) -> LayeredGeometry:
    """Fekanex: attention behind short convolutions with a rotation, unit q / k norms, a window that keeps the first keys and
    a unit sink; dense (clamped GLU) or mixture-of-experts (softmax over the chosen logits) feed-forwards beside the mixer
    under one norm; a hashed token-pair table added to the scaled embedding; logits from the embedding table, scaled."""
    layers = []
    for index, entry in enumerate(config["layers"]):
        m, kind = entry["mixer"], entry["type"]
        if kind != "attention":
            raise ValueError(f"unsupported mixer type {kind!r}; supported: attention")
        rot = RotarySpec.from_config(m["rot"]) if m.get("rot") else None
        mask = m.get("mask") or {}
        spec = MixerSpec("conv_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                         kv_heads=int(m.get("kv_heads") or m["heads"]), scale=float(m["scale"]), rotary=rot,
                         window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0), bias=True,
                         conv_taps=int(m.get("conv") or 0), unit_norm=True, unit_sink=True, value_mix=bool(m.get("v_mix")))
        if spec.heads % spec.kv_heads:
            raise ValueError(f"layer {index}: {spec.heads} query heads do not divide over {spec.kv_heads} key/value heads")
        if rot is not None and (rot.dims > spec.dim or rot.dims % 2):
            raise ValueError(f"layer {index}: {rot.dims} rotated entries do not fit heads of {spec.dim}")
        mlp = entry.get("mlp")
        if mlp is None:
            mspec = None
        elif mlp.get("kind", "dense") == "dense":
            mspec = MlpSpec("dense", ff=int(mlp["ff"]), act="clamped", limit=float(mlp["limit"]))
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            mspec = MlpSpec("moe", ff=int(mlp["expert"]["ff"]), act="silu", experts=int(r["experts"]), top=int(r["top"]),
                            scoring="softmax_chosen")
            if not 1 <= mspec.top <= mspec.experts:
                raise ValueError(f"layer {index}: {mspec.top} of {mspec.experts} experts cannot be chosen")
        else:
            raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}; supported: dense, moe")
        layers.append(LayerSpec(spec, ff=mspec.ff if mspec else 0, mlp_kind=mspec.kind if mspec else "dense", mlp=mspec))
    emb = config.get("embedding") or {}
    pair = emb.get("bigram") or {}
    return LayeredGeometry(name=name, vocab_size=int(config["vocab"]), width=int(config["width"]), eps=float(config["norm"]["eps"]),
                           layers=tuple(layers), token_shift=False, parallel=True, embed_scale=float(emb.get("scale", 1.0)),
                           pair_buckets=int(pair.get("buckets") or 0), pair_mul_prev=int(pair.get("mul_prev") or 0),
                           pair_mul_cur=int(pair.get("mul_cur") or 0), logit_scale=float(config.get("logit_scale", 1.0)),
                           tied_head=True)


def _nivotar_geometry(config: Mapping, name: str, shapes: Mapping) -> LayeredGeometry:
    """Nivotar: per layer one of three mixers -- ``parallel`` (windowed attention with whole-row q / k norms and a half-split
    rotation, beside a state-space mixer), ``lightning`` (linear attention with a fixed decay per head), ``gla`` (linear
    attention with a decay per key entry) --, a dense biased silu feed-forward or experts chosen by a corrected softmax score
    (some router outputs standing for the input itself), the norm on every sublayer's result, logits from the embedding
    table.  The width of the low-rank projection in front of a ``gla`` layer's decay logits is the row count of its ``mix.a1``
    tensor (``shapes``), or ``mixer.rank`` where a configuration is built without a checkpoint."""
    layers = []
    for index, entry in enumerate(config["layers"]):
        m, kind = entry["mixer"], entry["type"]
        if kind == "parallel":
            a, r = m["left"], m["right"]
            rot = RotarySpec(int(a["rot"]["dims"]), float(a["rot"]["base"])) if a.get("rot") else None
            ssd = StateSpaceSpec(heads=int(r["heads"]), vdim=int(r["vdim"]), state=int(r["state"]), groups=int(r["groups"]),
                                 conv_taps=int(r["conv"]), norm_groups=int(r["norm_groups"]))
            spec = MixerSpec("attention_ssd", heads=int(a["heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                             kv_heads=int(a.get("kv_heads") or a["heads"]), scale=float(a["scale"]), rotary=rot,
                             window=int((a.get("mask") or {}).get("size") or 0), ssd=ssd,
                             branch_scales=(float(m["left_scale"]), float(m["right_scale"])))
            if spec.heads % spec.kv_heads:
                raise ValueError(f"layer {index}: {spec.heads} query heads do not divide over {spec.kv_heads} key/value heads")
            if rot is not None and (rot.dims > spec.dim or rot.dims % 2):
                raise ValueError(f"layer {index}: {rot.dims} rotated entries do not fit heads of {spec.dim}")
            if ssd.heads % ssd.groups or ssd.inner % ssd.norm_groups or ssd.conv_taps < 1:
                raise ValueError(f"layer {index}: {ssd.heads} state-space heads of {ssd.vdim} do not divide over {ssd.groups} groups "
                                 f"/ {ssd.norm_groups} norm parts")
        elif kind == "lightning":
            spec = MixerSpec("decay_linear", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                             decay=tuple(float(d) for d in m["decay"]))
            if len(spec.decay) != spec.heads:
                raise ValueError(f"layer {index}: {len(spec.decay)} decays for {spec.heads} heads")
        elif kind == "gla":
            shape = shapes.get(f"l{index}.mix.a1")
            rank = int(shape[0]) if shape is not None else int(m.get("rank") or 0)
            spec = MixerSpec("gla", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), tau=float(m["tau"]), decay_rank=rank)
            if not spec.tau > 0 or rank < 1:
                raise ValueError(f"layer {index}: tau must be positive, and the decay projection's rank known (tensor mix.a1)")
        else:
            raise ValueError(f"unsupported mixer type {kind!r}; supported: parallel, lightning, gla")
        mlp = entry.get("mlp")
        if mlp is None:
            mspec = None
        elif mlp.get("kind", "dense") == "dense":
            mspec = MlpSpec("dense", ff=int(mlp["ff"]), act="silu", bias=True)
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            mspec = MlpSpec("moe", ff=int(mlp["expert"]["ff"]), act="clamped", limit=float(mlp["expert"]["limit"]),
                            experts=int(r["experts"]), top=int(r["top"]), scoring="softmax_all", identity=int(r.get("identity") or 0))
            if not 1 <= mspec.top <= mspec.experts + mspec.identity or mspec.experts < 1 or mspec.limit < 0:
                raise ValueError(f"layer {index}: {mspec.top} of {mspec.experts} + {mspec.identity} experts cannot be chosen")
        else:
            raise ValueError(f"unsupported feed-forward kind {mlp.get('kind')!r}; supported: dense, moe")
        layers.append(LayerSpec(spec, ff=mspec.ff if mspec else 0, mlp_kind=mspec.kind if mspec else "dense", mlp=mspec))
    return LayeredGeometry(name=name, vocab_size=int(config["vocab"]), width=int(config["width"]), eps=float(config["norm"]["eps"]),
                           layers=tuple(layers), token_shift=False, tied_head=True, post_norm=True)


def _linear(inp: int, out: int) -> ReplicatedLinear:
    return ReplicatedLinear(inp, out)


def _vector(n: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(n, dtype=torch.float16), requires_grad=False)


# ------------------------------------------------------------------------------------- #
# mixers
# ------------------------------------------------------------------------------------- #
class SinkAttention(nn.Module):
    """``q|k|v`` in one projection, then per-head norm + temperature + cache write (one launch), attention with a sink over
    the paged cache (one launch), output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        self.q_size, self.k_size, self.v_size = spec.heads * spec.dim, spec.kv_heads * spec.dim, spec.kv_heads * spec.vdim
        self.qkv_proj = _linear(width, self.q_size + self.k_size + self.v_size)
        self.o_proj = _linear(spec.heads * spec.vdim, width)
        self.q_norm_weight = _vector(spec.dim)
        self.k_norm_weight = _vector(spec.dim)
        self.sink = _vector(spec.heads)

    def cache_run(self) -> dict:
        return {"kind": "attention", "kv_heads": self.spec.kv_heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s = self.spec
        k_cache, v_cache = cache.kv_buffer[run]
        q = qk_norm_cache(self.qkv_proj(h), s.heads, s.kv_heads, s.dim, s.vdim, self.q_norm_weight, self.k_norm_weight, self.eps,
                          s.temp_coef, s.temp_every, step, k_cache, v_cache)
        o = ragged_attention(q, k_cache, v_cache, s.scale, step, token_table, sink=self.sink)
        return self.o_proj(o)


class GatedLinearMixer(nn.Module):
    """HGRN2.  ``q|f|v`` in one projection; gate, recurrence, read-out and the per-head output norm in one launch over the
    fp32 state slots; output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        self.qk_size, self.v_size = spec.heads * spec.dim, spec.heads * spec.vdim
        self.qfv_proj = _linear(width, 2 * self.qk_size + self.v_size)
        self.o_proj = _linear(self.v_size, width)
        self.f_bias = _vector(self.qk_size)
        self.lower = _vector(self.qk_size)
        self.out_norm_weight = _vector(spec.vdim)

    def cache_run(self) -> dict:
        return {"kind": "recurrent", "heads": self.spec.heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s = self.spec
        o = gated_linear_scan(self.qfv_proj(h), s.heads, s.dim, s.vdim, self.f_bias, self.lower, self.out_norm_weight, self.eps,
                              step, cache.recurrent[run])
        return self.o_proj(o)


class DenseMLP(nn.Module):
    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up_proj = _linear(width, ff)
        self.down_proj = _linear(ff, width)
        self.act = _vector(2)

    def forward(self, h):
        return self.down_proj(xielu(self.up_proj(h), self.act))


class LatentAttention(nn.Module):
    """Attention whose keys and values are up-projections of ONE cached latent row per token, plus a rotated key part that
    all heads share.  The cache is read in the absorbed form: it holds ``[latent | rotated key part]`` (one key/value head of
    key width ``kv_rank + rot_dim``; the values are the first ``kv_rank`` columns of the same rows), a head's query becomes
    ``[W_uk^T q_unrotated | rotate(q_rotated)]`` and its output ``W_uv (weights . latents)`` -- two batched products over the
    heads around the attention kernel.  Whole prompts (every sequence of the step at position 0) need nothing from the cache
    and expand keys and values per head from the step's own rows instead (:meth:`_expanded`).  Everything that reads the
    mixer's input (query or query latent, key/value latent, output gate, ``extra`` columns of the layer) is one projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float, extra: int = 0):
        super().__init__()
        self.spec, self.eps, self.extra = spec, eps, extra
        s = spec
        self.q_width = s.heads * (s.dim + s.rot_dim)
        q_cols = s.q_rank if s.q_rank else self.q_width
        self.kv_off = q_cols
        self.gate_off = q_cols + s.kv_rank + s.rot_dim
        self.extra_off = self.gate_off + (s.heads * s.vdim if s.out_gate else 0)
        self.in_proj = _linear(width, self.extra_off + extra)
        if s.q_rank:
            self.q_norm_weight = _vector(s.q_rank)
            self.uq_proj = _linear(s.q_rank, self.q_width)
        self.kv_norm_weight = _vector(s.kv_rank)
        self.uk_weight = nn.Parameter(torch.zeros(s.heads * s.dim, s.kv_rank, dtype=torch.float16), requires_grad=False)
        self.uv_weight = nn.Parameter(torch.zeros(s.heads * s.vdim, s.kv_rank, dtype=torch.float16), requires_grad=False)
        self.o_proj = _linear(s.heads * s.vdim, width)
        self._freq_values, self.amp = s.rotary.table()
        self.pairs = len(self._freq_values)
        self._freq = None   # fp32 on the device of the first step (not a buffer: a module-wide cast must not touch the angles)

    def cache_run(self) -> dict:
        return {"kind": "latent", "rank": self.spec.kv_rank, "rot": self.spec.rot_dim}

    # whole prompts of at least this many tokens take the expanded form (keys / values per head from the step's own latents)
    expand_min_run = 64

    def forward(self, h, step, cache, run: int, token_table):
        s = self.spec
        n = h.shape[0]
        rows = self.in_proj(h)
        k_cache, v_cache = cache.kv_buffer[run]
        if self._freq is None or self._freq.device != h.device:
            self._freq = torch.tensor(self._freq_values, dtype=torch.float64).to(torch.float32).to(h.device)
        cache_rows = k_cache.view(k_cache.shape[0], -1)
        c_q = latent_kv_prep(rows, self.kv_off, s.kv_rank, s.rot_dim, self.kv_norm_weight, self.eps, self._freq, self.pairs, self.amp,
                             step, cache_rows, q_off=0, q_rank=s.q_rank, q_norm_weight=self.q_norm_weight if s.q_rank else None)
        q = (self.uq_proj(c_q) if s.q_rank else rows[:, :self.q_width]).view(n, s.heads, s.dim + s.rot_dim)
        if step.all_start and step.longest_run >= self.expand_min_run:
            o = self._expanded(q, cache_rows, step)
        else:
            o = self._absorbed(q, k_cache, v_cache, step, token_table)
        if s.out_gate:
            o = glu_act(rows[:, self.gate_off:], s.heads * s.vdim, "sigmoid", up=o)
        return self.o_proj(o), (rows[:, self.extra_off:] if self.extra else None)

    def _absorbed(self, q, k_cache, v_cache, step, token_table):
        """Any step: queries against the cached latent rows."""
        s, n = self.spec, q.shape[0]
        qa = torch.empty(n, s.heads, s.kv_rank + s.rot_dim, dtype=q.dtype, device=q.device)
        # absorbed query: [heads, n, dim] x [heads, dim, rank] straight into the front columns of the query rows
        torch.bmm(q[:, :, :s.dim].transpose(0, 1), self.uk_weight.view(s.heads, s.dim, s.kv_rank),
                  out=qa[:, :, :s.kv_rank].transpose(0, 1))
        rotate_pairs(q, s.dim, s.rot_dim, self._freq, self.pairs, self.amp, step, qa, s.kv_rank)
        o_lat = ragged_attention(qa, k_cache, v_cache, s.scale, step, token_table, window=s.window)     # [n, heads * rank]
        o = torch.empty(n, s.heads, s.vdim, dtype=q.dtype, device=q.device)
        torch.bmm(o_lat.view(n, s.heads, s.kv_rank).transpose(0, 1), self.uv_weight.view(s.heads, s.vdim, s.kv_rank).transpose(1, 2),
                  out=o.transpose(0, 1))
        return o.view(n, s.heads * s.vdim)

    def _expanded(self, q, cache_rows, step):
        """A step in which every sequence starts at position 0 (whole prompts): all keys a token may see are tokens of this
        step, so keys ``[W_uk c | rotated part]`` and values ``W_uv c`` are expanded per head from the rows the step has just
        written, and attention runs with the heads' own narrow widths (dim + rot_dim, vdim) instead of rank + rot_dim, rank:
        a fraction of the absorbed form's work per (query, key) pair.  Same values up to rounding."""
        s, n = self.spec, q.shape[0]
        written = cache_rows.index_select(0, step.select.long())                        # [n, rank + rot]: normed latent | rotated part
        latent = written[:, :s.kv_rank]
        if q.is_contiguous():
            qf = q
        else:
            qf = q.contiguous()
        rotate_pairs(qf, s.dim, s.rot_dim, self._freq, self.pairs, self.amp, step, qf, s.dim)             # (in place)
        keys = torch.empty(n, s.heads, s.dim + s.rot_dim, dtype=q.dtype, device=q.device)
        keys[:, :, :s.dim] = torch.nn.functional.linear(latent, self.uk_weight).view(n, s.heads, s.dim)
        keys[:, :, s.dim:] = written[:, None, s.kv_rank:]
        values = torch.nn.functional.linear(latent, self.uv_weight).view(n, s.heads, s.vdim)
        # the step's own tokens as a cache: sequence i of the step owns rows seq_start[i] .. ; positions are row offsets
        own = torch.arange(step.num_seqs, dtype=torch.int32, device=q.device)
        table = (step.seq_start[:-1, None] + torch.arange(step.longest_run, dtype=torch.int32, device=q.device)[None, :]).contiguous()
        local = dataclasses.replace(step, seq_slot=own)
        return ragged_attention(qf, keys, values, s.scale, local, table, window=s.window)


class MinGRU(nn.Module):
    """``z | x | g`` (and ``extra`` columns of the layer) in one projection; gates, recurrence and the silu-gated read-out in
    one launch over the fp32 state slots; output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float, extra: int = 0):
        super().__init__()
        self.spec, self.extra = spec, extra
        self.in_proj = _linear(width, 3 * spec.width + extra)
        self.z_bias = _vector(spec.width)
        self.x_bias = _vector(spec.width)
        self.o_proj = _linear(spec.width, width)

    def cache_run(self) -> dict:
        return {"kind": "recurrent", "heads": 1, "dk": 1, "dv": self.spec.width}

    def forward(self, h, step, cache, run: int, token_table):
        w = self.spec.width
        rows = self.in_proj(h)
        o = mingru_scan(rows, w, self.z_bias, self.x_bias, step, cache.recurrent[run].view(-1, w))
        return self.o_proj(o), (rows[:, 3 * w:] if self.extra else None)


class GatedMLP(nn.Module):
    """``down(act(gate h) * (up h))``; ``gate | up`` (and ``extra`` columns of the layer) are one projection."""

    def __init__(self, width: int, ff: int, act: str, extra: int = 0):
        super().__init__()
        self.ff, self.act, self.extra = ff, act, extra
        self.in_proj = _linear(width, 2 * ff + extra)
        self.down_proj = _linear(ff, width)

    def forward(self, h):
        rows = self.in_proj(h)
        return self.down_proj(glu_act(rows, self.ff, self.act)), (rows[:, 2 * self.ff:] if self.extra else None), None, None


class SparseMoE(nn.Module):
    """Sigmoid router over expert groups (fp32), the chosen experts' gated feed-forwards as grouped products over slots sorted
    by expert, and a shared expert whose result is scaled per token by ``sigmoid(w_sg . h)``.  The slots' rows are NOT summed
    here: they ride, with the shared row and its scale, into the norm launch that follows."""

    def __init__(self, width: int, spec: MlpSpec, extra: int = 0):
        super().__init__()
        self.spec, self.extra = spec, extra
        self.router_weight = nn.Parameter(torch.zeros(spec.experts, width, dtype=torch.float16), requires_grad=False)
        self.gate_up_weight = nn.Parameter(torch.zeros(spec.experts, 2 * spec.ff, width, dtype=torch.float16), requires_grad=False)
        self.down_weight = nn.Parameter(torch.zeros(spec.experts, width, spec.ff, dtype=torch.float16), requires_grad=False)
        if spec.shared_ff or extra:
            self.in_proj = _linear(width, 2 * spec.shared_ff + extra)   # shared gate | shared up | the layer's columns
        if spec.shared_ff:
            self.shared_down_proj = _linear(spec.shared_ff, width)
            self.shared_scale_weight = nn.Parameter(torch.zeros(1, width, dtype=torch.float16), requires_grad=False)

    def forward(self, h):
        s = self.spec
        ids, weights, scale = group_router(h, self.router_weight, s.top, s.group_count, s.group_keep, s.route_scale,
                                           extra_weight=self.shared_scale_weight if s.shared_ff else None)
        y = sparse_glu_experts(h, self.gate_up_weight, self.down_weight, ids, weights)
        rows = self.in_proj(h) if (s.shared_ff or self.extra) else None
        shared = self.shared_down_proj(glu_act(rows, s.shared_ff, "silu")) if s.shared_ff else None
        return y, (rows[:, 2 * s.shared_ff:] if self.extra else None), shared, scale


class ConvRotaryAttention(nn.Module):
    """``q | k | v`` (and ``extra`` columns of the layer) in one projection; bias, convolution over time, rotation, unit q / k
    norms, value blend and the cache write in one launch; attention over the paged cache with a window, kept first keys and a
    sink of score 0.  The heads' outputs go to ``out`` (a column range of the layer's output projection input): the output
    projection is the layer's."""

    def __init__(self, width: int, spec: MixerSpec, eps: float, extra: int = 0):
        super().__init__()
        self.spec, self.eps, self.extra = spec, eps, extra
        s = spec
        self.channels = (s.heads + s.kv_heads) * s.dim + s.kv_heads * s.vdim
        self.in_proj = _linear(width, self.channels + extra)
        self.qkv_bias = _vector(self.channels) if s.bias else None
        self.conv_weight = (nn.Parameter(torch.zeros(self.channels, s.conv_taps, dtype=torch.float16), requires_grad=False)
                            if s.conv_taps else None)
        self.value_blend = _vector(1) if s.value_mix else None
        self._freq_values, self.amp = s.rotary.table() if s.rotary is not None else ([], 1.0)
        self.pairs = len(self._freq_values)
        self._freq = None   # fp32 on the device of the first step (not a buffer: a module-wide cast must not touch the angles)
        self._sink = None   # zeros [heads]: exp(0) = 1 in every denominator

    def cache_run(self) -> dict:
        s = self.spec
        return {"kind": "attention", "kv_heads": s.kv_heads, "dk": s.dim, "dv": s.vdim, "conv_taps": s.conv_taps,
                "conv_channels": self.channels, "value_mix": s.value_mix}

    def forward(self, h, step, cache, run: int, token_table, out=None):
        s = self.spec
        rows = self.in_proj(h)
        k_cache, v_cache = cache.kv_buffer[run]
        if self.pairs and (self._freq is None or self._freq.device != h.device):
            self._freq = torch.tensor(self._freq_values, dtype=torch.float64).to(torch.float32).to(h.device)
        if s.unit_sink and (self._sink is None or self._sink.device != h.device or self._sink.dtype != h.dtype):
            self._sink = torch.zeros(s.heads, dtype=h.dtype, device=h.device)
        source = cache.value_source[run]
        table = None
        if self.pairs:   # cos / sin per token: once per step for all layers that rotate alike
            key = ("rotation", self.pairs, self.amp, tuple(self._freq_values))
            shared = getattr(step, "shared", None)
            table = shared.get(key) if shared is not None else None
            if table is None:
                table = rotation_table(step, self._freq, self.pairs, self.amp)
                if shared is not None:
                    shared[key] = table
        q = conv_rope_cache(rows, s.heads, s.kv_heads, s.dim, s.vdim, step, k_cache, v_cache, bias=self.qkv_bias,
                            conv_weight=self.conv_weight, conv_state=cache.conv[run], freq=self._freq, pairs=self.pairs,
                            amp=self.amp, unit_norm=s.unit_norm, eps=self.eps,
                            v_source=cache.kv_buffer[source][1] if source is not None else None,
                            v_blend=self.value_blend if source is not None else None, rot_table=table)
        o = ragged_attention(q, k_cache, v_cache, s.scale, step, token_table, sink=self._sink if s.unit_sink else None,
                             window=s.window, keep_first=s.keep_first, out=out)
        return o, (rows[:, self.channels:] if self.extra else None)


class ChosenSoftmaxMoE(nn.Module):
    """The ``top`` largest router logits (fp32) choose a token's experts; their weights are the softmax over the chosen logits
    alone.  Experts are gated feed-forwards without biases, run as grouped products over slots sorted by expert.  The slots'
    rows are NOT summed here: they ride into the norm launch that follows."""

    def __init__(self, width: int, spec: MlpSpec):
        super().__init__()
        self.spec = spec
        self.router_weight = nn.Parameter(torch.zeros(spec.experts, width, dtype=torch.float16), requires_grad=False)
        self.gate_up_weight = nn.Parameter(torch.zeros(spec.experts, 2 * spec.ff, width, dtype=torch.float16), requires_grad=False)
        self.down_weight = nn.Parameter(torch.zeros(spec.experts, width, spec.ff, dtype=torch.float16), requires_grad=False)

    def forward(self, h):
        ids, weights, _ = group_router(h, self.router_weight, self.spec.top, scoring=self.spec.scoring)
        return sparse_glu_experts(h, self.gate_up_weight, self.down_weight, ids, weights)


class WindowAttentionSSD(nn.Module):
    """Two mixers side by side on the same input, ``a_l * attention(h) + a_r * ssd(h)``, with ONE input projection
    ``q | k | v | z | u B C | dt`` and ONE output projection ``[W_o,left | W_o,right]`` over ``[a_l * heads' outputs | a_r *
    gated, normed read-out]``, whose fp32 accumulation is the sum of the branches.  Attention: q and k RMS-normed over their
    whole rows, rotated in (i, i + dims / 2) pairs, a sliding window over the paged cache (``a_l`` rides on the cached values).
    State-space branch: ``u B C`` through a causal convolution and silu, then per head ``S <- exp(-exp(A_log) dt) S + dt B u^T``,
    ``y = S^T C + D u`` (B, C shared by the heads of a group), ``y silu(z)`` RMS-normed in equal parts."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        s, r = spec, spec.ssd
        self.qkv = (s.heads + s.kv_heads) * s.dim + s.kv_heads * s.vdim
        self.z_off = self.qkv
        self.conv_off = self.z_off + r.inner
        self.dt_off = self.conv_off + r.conv_channels
        self.in_proj = _linear(width, self.dt_off + r.heads)
        self.q_norm_weight = _vector(s.heads * s.dim)
        self.k_norm_weight = _vector(s.kv_heads * s.dim)
        self.conv_weight = nn.Parameter(torch.zeros(r.conv_channels, r.conv_taps, dtype=torch.float16), requires_grad=False)
        self.conv_bias = _vector(r.conv_channels)
        self.dt_bias, self.a_log, self.skip = _vector(r.heads), _vector(r.heads), _vector(r.heads)
        self.ssd_norm_weight = _vector(r.inner)
        self.heads_width = s.heads * s.vdim
        self.out_proj = _linear(self.heads_width + r.inner, width)
        self._freq_values = s.rotary.table()[0] if s.rotary is not None else []
        self.pairs = len(self._freq_values)
        self._freq = None   # fp32 on the device of the first step (not a buffer: a module-wide cast must not touch the angles)

    def cache_run(self) -> dict:
        s, r = self.spec, self.spec.ssd
        return {"kind": "attention", "kv_heads": s.kv_heads, "dk": s.dim, "dv": s.vdim, "state": (r.heads, r.state, r.vdim),
                "conv_taps": r.conv_taps, "conv_channels": r.conv_channels}

    def forward(self, h, step, cache, run: int, token_table):
        s, r = self.spec, self.spec.ssd
        rows = self.in_proj(h)
        if self.pairs and (self._freq is None or self._freq.device != h.device):
            self._freq = torch.tensor(self._freq_values, dtype=torch.float64).to(torch.float32).to(h.device)
        mixed = torch.empty(h.shape[0], self.heads_width + r.inner, dtype=h.dtype, device=h.device)
        k_cache, v_cache = cache.kv_buffer[run]
        q = rownorm_rope_cache(rows, s.heads, s.kv_heads, s.dim, s.vdim, step, k_cache, v_cache, q_weight=self.q_norm_weight,
                               k_weight=self.k_norm_weight, eps=self.eps, freq=self._freq, pairs=self.pairs,
                               value_scale=s.branch_scales[0])
        ragged_attention(q, k_cache, v_cache, s.scale, step, token_table, window=s.window, out=mixed[:, :self.heads_width])
        ubc = conv_act(rows[:, self.conv_off:self.dt_off], self.conv_weight, self.conv_bias, step, cache.conv[run])
        gn = r.groups * r.state
        o = linear_scan(ubc[:, r.inner + gn:], ubc[:, r.inner:r.inner + gn], ubc[:, :r.inner], r.heads, r.state, r.vdim, step,
                        cache.recurrent[run], qk_heads=r.groups, dt=rows[:, self.dt_off:], dt_bias=self.dt_bias, a_log=self.a_log,
                        skip=self.skip)
        gated_out_norm(o, self.ssd_norm_weight, self.eps, parts=r.norm_groups, gate=rows[:, self.z_off:self.conv_off],
                       gate_kind="silu", gate_first=True, scale=s.branch_scales[1], out=mixed[:, self.heads_width:])
        return self.out_proj(mixed)


class DecayLinearAttention(nn.Module):
    """``q | k | v | g`` in one projection; per head ``S <- decay_h S + silu(k) silu(v)^T``, ``o = S^T silu(q)`` over the fp32
    state slots; the heads side by side RMS-normed together, times ``sigmoid(g)``; output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        self.qk, self.v = spec.heads * spec.dim, spec.heads * spec.vdim
        self.in_proj = _linear(width, 2 * self.qk + 2 * self.v)
        self.out_norm_weight = _vector(self.v)
        self.o_proj = _linear(self.v, width)
        self._decay = None   # fp32 on the device of the first step (not a buffer: a module-wide cast must not round the decays)

    def cache_run(self) -> dict:
        return {"kind": "recurrent", "heads": self.spec.heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s, qk, v = self.spec, self.qk, self.v
        rows = self.in_proj(h)
        if self._decay is None or self._decay.device != h.device:
            self._decay = torch.tensor(s.decay, dtype=torch.float64).to(torch.float32).to(h.device)
        o = linear_scan(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + v], s.heads, s.dim, s.vdim, step,
                        cache.recurrent[run], act=True, head_decay=self._decay)
        return self.o_proj(gated_out_norm(o, self.out_norm_weight, self.eps, gate=rows[:, 2 * qk + v:], gate_kind="sigmoid"))


class GatedLinearAttention(nn.Module):
    """``q | k | v | g | a`` in one projection (``a``: the low-rank input of the decay logits); per head
    ``S <- diag(alpha) S + k v^T``, ``o = S^T q / sqrt(dim)`` with ``alpha = sigmoid(W_a2 a + b)^(1 / tau)`` per key entry;
    every head RMS-normed with one shared weight, times ``silu(g)``; output projection."""

    def __init__(self, width: int, spec: MixerSpec, eps: float):
        super().__init__()
        self.spec, self.eps = spec, eps
        rank = spec.decay_rank
        self.qk, self.v = spec.heads * spec.dim, spec.heads * spec.vdim
        self.in_proj = _linear(width, 2 * self.qk + 2 * self.v + rank)
        self.decay_proj = _linear(rank, self.qk)
        self.decay_bias = _vector(self.qk)
        self.out_norm_weight = _vector(spec.vdim)
        self.o_proj = _linear(self.v, width)

    def cache_run(self) -> dict:
        return {"kind": "recurrent", "heads": self.spec.heads, "dk": self.spec.dim, "dv": self.spec.vdim}

    def forward(self, h, step, cache, run: int, token_table):
        s, qk, v = self.spec, self.qk, self.v
        rows = self.in_proj(h)
        logits = self.decay_proj(rows[:, 2 * qk + 2 * v:].contiguous())
        o = linear_scan(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + v], s.heads, s.dim, s.vdim, step,
                        cache.recurrent[run], q_scale=s.dim ** -0.5, gate=logits, gate_bias=self.decay_bias, tau=s.tau)
        return self.o_proj(gated_out_norm(o, self.out_norm_weight, self.eps, parts=s.heads, gate=rows[:, 2 * qk + v:2 * qk + 2 * v],
                                          gate_kind="silu"))


class BiasedGatedMLP(nn.Module):
    """``down(silu(gate h + b_g) * (up h + b_u)) + b_d``; ``gate | up`` are one projection.  The down projection's bias is
    not added here: it rides with the result into the norm launch that follows."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.ff = ff
        self.in_proj = ReplicatedLinear(width, 2 * ff, bias=True)
        self.down_proj = _linear(ff, width)
        self.down_bias = _vector(width)

    def forward(self, h):
        return self.down_proj(glu_act(self.in_proj(h), self.ff, "silu")), self.down_bias, None, None


class CorrectedSoftmaxMoE(nn.Module):
    """Scores are the softmax (fp32) over ALL router outputs; the ``top`` largest ``score + correction`` choose, the scores
    alone weigh (not renormalised).  Experts are clamped gated feed-forwards without biases, run as grouped products over slots
    sorted by expert.  The last ``identity`` router outputs have no weights: a token that chooses one gets its own input row
    times the score.  Neither the slots' rows nor that row are summed here: they ride into the norm launch that follows."""

    def __init__(self, width: int, spec: MlpSpec):
        super().__init__()
        self.spec = spec
        outputs = spec.experts + spec.identity
        self.router_weight = nn.Parameter(torch.zeros(outputs, width, dtype=torch.float16), requires_grad=False)
        self.correction = _vector(outputs)
        self.gate_up_weight = nn.Parameter(torch.zeros(spec.experts, 2 * spec.ff, width, dtype=torch.float16), requires_grad=False)
        self.down_weight = nn.Parameter(torch.zeros(spec.experts, width, spec.ff, dtype=torch.float16), requires_grad=False)

    def forward(self, h):
        s = self.spec
        ids, weights, own = group_router(h, self.router_weight, s.top, scoring=s.scoring, correction=self.correction,
                                         identity=s.identity)
        y = sparse_glu_experts(h, self.gate_up_weight, self.down_weight, ids, weights, limit=s.limit, skipped_ids=s.identity > 0)
        return y, None, (h if s.identity else None), own


MIXERS = {"attention": SinkAttention, "hgrn2": GatedLinearMixer, "latent_attention": LatentAttention, "mingru": MinGRU,
          "conv_attention": ConvRotaryAttention, "attention_ssd": WindowAttentionSSD, "decay_linear": DecayLinearAttention,
          "gla": GatedLinearAttention}


class MixerLayer(nn.Module):
    def __init__(self, geo: LayeredGeometry, spec: LayerSpec):
        super().__init__()
        self.eps = geo.eps
        self.norm1_weight = _vector(geo.width)
        self.shift = _vector(geo.width) if geo.token_shift else None
        self.mixer = MIXERS[spec.mixer.kind](geo.width, spec.mixer, geo.eps)
        self.mlp = DenseMLP(geo.width, spec.ff) if spec.ff else None
        self.norm2_weight = _vector(geo.width) if spec.ff else None

    def forward(self, x, delta, step, cache, run: int, token_table):
        """``(x, delta)``: the fp32 residual and the update still to be added to it.  Returns the same pair."""
        h, x = add_rmsnorm_shift(x, delta, self.norm1_weight, self.eps, shift=self.shift, step=step, state=cache.shift[run])
        delta = self.mixer(h, step, cache, run, token_table)
        if self.mlp is not None:
            h, x = add_rmsnorm_shift(x, delta, self.norm2_weight, self.eps, x_out=x)
            delta = self.mlp(h)
        return x, delta


class SandwichLayer(nn.Module):
    """``x <- x + norm_b(f(norm_a(x)) * sigmoid(W_r norm_a(x) + b_r))`` for the mixer and then for the feed-forward, norms
    over groups.  ``W_r`` rides as extra columns in the sublayer's input projection; a sublayer's result is carried as a
    :class:`GatedUpdate` into the norm launch that opens the next sublayer (gate, post-norm, residual add and pre-norm are one
    launch)."""

    def __init__(self, geo: LayeredGeometry, spec: LayerSpec):
        super().__init__()
        self.eps, self.groups = geo.eps, geo.norm_groups
        w = geo.width
        self.norm1_weight, self.norm1b_weight = _vector(w), _vector(w)
        self.rg1_bias = _vector(w)
        self.mixer = MIXERS[spec.mixer.kind](w, spec.mixer, geo.eps, extra=w)
        self.mlp = None
        if spec.mlp is not None:
            self.norm2_weight, self.norm2b_weight = _vector(w), _vector(w)
            self.rg2_bias = _vector(w)
            self.mlp = SparseMoE(w, spec.mlp, extra=w) if spec.mlp.kind == "moe" else GatedMLP(w, spec.mlp.ff, spec.mlp.act, extra=w)

    def forward(self, x, pending, step, cache, run: int, token_table):
        """``(x, pending)``: the fp32 residual (updated in place) and the update still to enter it.  Returns the same pair."""
        h = gated_group_norm(x, pending, self.norm1_weight, self.eps, self.groups)
        y, gate = self.mixer(h, step, cache, run, token_table)
        pending = GatedUpdate(y, self.norm1b_weight, gate, self.rg1_bias)
        if self.mlp is not None:
            h = gated_group_norm(x, pending, self.norm2_weight, self.eps, self.groups)
            y, gate, shared, scale = self.mlp(h)
            pending = GatedUpdate(y, self.norm2b_weight, gate, self.rg2_bias, shared, scale)
        return x, pending


class ParallelLayer(nn.Module):
    """``x <- x + (mixer(h) + feed_forward(h))`` with ``h = norm(x)``: one norm, both sublayers read it.  With a dense
    feed-forward, ``q | k | v | gate | up`` are ONE input projection and ``[heads' outputs | activation]`` go through ONE output
    projection ``[W_o | W_down]``, whose fp32 accumulation is the sum of the two sublayers.  With experts, the mixer's output
    projection gives one row and the experts' slots ride beside it as a :class:`SummedUpdate` into the next norm launch."""

    slope = 1.702   # inside the sigmoid of the clamped GLU

    def __init__(self, geo: LayeredGeometry, spec: LayerSpec):
        super().__init__()
        self.eps = geo.eps
        w, m = geo.width, spec.mixer
        self.norm1_weight = _vector(w)
        self.dense = spec.mlp if (spec.mlp is not None and spec.mlp.kind == "dense") else None
        ff = self.dense.ff if self.dense is not None else 0
        self.mixer = MIXERS[m.kind](w, m, geo.eps, extra=2 * ff)
        self.heads_width = m.heads * m.vdim
        self.out_proj = _linear(self.heads_width + ff, w)
        self.experts = ChosenSoftmaxMoE(w, spec.mlp) if (spec.mlp is not None and spec.mlp.kind == "moe") else None

    def forward(self, x, pending, step, cache, run: int, token_table):
        """``(x, pending)``: the fp32 residual (updated in place) and the update still to enter it.  Returns the same pair."""
        h, x = add_rmsnorm_shift(x, pending, self.norm1_weight, self.eps, x_out=x)
        ff = self.dense.ff if self.dense is not None else 0
        mixed = torch.empty(h.shape[0], self.heads_width + ff, dtype=h.dtype, device=h.device)
        _, gate_up = self.mixer(h, step, cache, run, token_table, out=mixed[:, :self.heads_width])
        if ff:
            glu_act(gate_up, ff, self.dense.act, limit=self.dense.limit, slope=self.slope, out=mixed[:, self.heads_width:])
        row = self.out_proj(mixed)
        return x, SummedUpdate(row, self.experts(h) if self.experts is not None else None)


class PostNormLayer(nn.Module):
    """``x <- x + norm_1(mixer(x))``, then ``x <- x + norm_2(feed_forward(x))``: sublayers read the residual stream itself (cast
    to the storage dtype), the norm sits on each sublayer's RESULT.  A result is carried as a :class:`GatedUpdate` into the
    launch that opens the next sublayer: norm of the result, residual add and the cast of the new stream are one launch."""

    def __init__(self, geo: LayeredGeometry, spec: LayerSpec):
        super().__init__()
        self.eps = geo.eps
        w, m = geo.width, spec.mixer
        self.norm1_weight = _vector(w)
        self.mixer = MIXERS[m.kind](w, m, geo.eps)
        self.mlp = None
        if spec.mlp is not None:
            self.norm2_weight = _vector(w)
            self.mlp = CorrectedSoftmaxMoE(w, spec.mlp) if spec.mlp.kind == "moe" else BiasedGatedMLP(w, spec.mlp.ff)

    def forward(self, x, pending, step, cache, run: int, token_table):
        """``(x, pending)``: the fp32 residual (updated in place) and the update still to enter it.  Returns the same pair."""
        dt = self.norm1_weight.dtype
        h = gated_group_norm(x, pending, None, self.eps, plain=dt)
        pending = GatedUpdate(self.mixer(h, step, cache, run, token_table), self.norm1_weight)
        if self.mlp is not None:
            h = gated_group_norm(x, pending, None, self.eps, plain=dt)
            y, bias, own, own_scale = self.mlp(h)
            pending = GatedUpdate(y, self.norm2_weight, shared=own, shared_scale=own_scale, bias=bias)
        return x, pending


# ------------------------------------------------------------------------------------- #
# the model
# ------------------------------------------------------------------------------------- #
class LayeredLM(nn.Module):
    """Token ids of a ragged step -> logits of the asked rows."""

    def __init__(self, geo: LayeredGeometry, dtype=torch.bfloat16):
        super().__init__()
        if get_tp_world_size() != 1:
            raise ValueError("layered models run on one GPU per replica (their projections are not sharded)")
        self.geo = geo
        self.embed_tokens = nn.Embedding(geo.vocab_size, geo.width, dtype=torch.float16)
        self.embed_tokens.weight.requires_grad_(False)
        make = SandwichLayer if geo.sandwich else ParallelLayer if geo.parallel else PostNormLayer if geo.post_norm else MixerLayer
        # a layer that borrows weights IS the other layer's module (which may come later in the stack); its cache run stays its own
        built = [make(geo, spec) if spec.weights_of is None else None for spec in geo.layers]
        self.layers = nn.ModuleList(built[i] if spec.weights_of is None else built[spec.weights_of] for i, spec in enumerate(geo.layers))
        if geo.looped:
            self.loop_in = _linear(2 * geo.width, geo.width)
            self.loop_step = nn.Parameter(torch.zeros(geo.loop_times, geo.width, dtype=torch.float16), requires_grad=False)
        self.norm_weight = _vector(geo.width)
        self.lm_head = _linear(geo.width, geo.vocab_size)
        if geo.tied_head:   # (one parameter: it is listed, loaded and cast as the embedding table)
            self.lm_head.weight = self.embed_tokens.weight
        if geo.pair_buckets:
            self.pair_table = nn.Parameter(torch.zeros(geo.pair_buckets + 1, geo.width, dtype=torch.float16), requires_grad=False)
        self.needs_previous_token = geo.pair_buckets > 0
        self.run_order = geo.run_order()
        self.to(dtype)

    @property
    def dtype(self):
        return self.norm_weight.dtype

    def cache_runs(self) -> list[dict]:
        """What every layer run keeps per sequence (the constructor argument of :class:`PagedStateCache`)."""
        runs = []
        for index, _, _ in self.run_order:
            layer = self.layers[index]
            run = layer.mixer.cache_run()
            if getattr(layer, "shift", None) is not None:
                run["shift_width"] = self.geo.width
            runs.append(run)
        return runs

    @torch.no_grad()
    def forward(self, token_ids, step, cache, token_table, logits_rows=None, collect_layers: list | None = None):
        """``token_ids [n]`` int64 of the step's flat token array.  ``logits_rows``: int64 indices into it (``None``: no
        logits, the step only fills cache and state).  ``collect_layers``: a list that receives the fp32 residual stream after
        every layer run (diagnostics; costs one add per run)."""
        if self.geo.pair_buckets or self.geo.embed_scale != 1.0:
            x0 = embed_pair(token_ids, self.embed_tokens.weight, self.geo.embed_scale, self.pair_table if self.geo.pair_buckets else None,
                            self.geo.pair_mul_prev, self.geo.pair_mul_cur, step, cache.prev_token)
        else:
            x0 = residual_set(F.embedding(token_ids, self.embed_tokens.weight))
        x, delta = (x0.clone() if self.geo.looped else x0), None  # (layers update the residual in place; x0 is read again)
        for run, (index, pass_no, first) in enumerate(self.run_order):
            if first:
                y = self.loop_in(cast_pair(x, x0, self.dtype, a_delta=delta))
                x, delta = residual_set(y, self.loop_step[pass_no]), None
            x, delta = self.layers[index](x, delta, step, cache, run, token_table)
            if collect_layers is not None:
                if self.geo.sandwich or self.geo.post_norm:   # (diagnostics: the pending update is applied to a copy)
                    seen = x.clone()
                    gated_group_norm(seen, delta, None, self.geo.eps, self.geo.norm_groups)
                    collect_layers.append(seen)
                elif isinstance(delta, SummedUpdate):
                    collect_layers.append(x + delta.total())
                else:
                    collect_layers.append(x + delta.float() if delta is not None else x.clone())
        if logits_rows is None:
            return None
        x = x[logits_rows].contiguous()
        if self.geo.sandwich or self.geo.post_norm:
            h = gated_group_norm(x, delta.rows(logits_rows) if delta is not None else None, self.norm_weight, self.geo.eps,
                                 self.geo.norm_groups)
        else:
            if isinstance(delta, SummedUpdate):
                delta = delta.rows(logits_rows)
            else:
                delta = delta[logits_rows].contiguous() if delta is not None else None
            h, _ = add_rmsnorm_shift(x, delta, self.norm_weight, self.geo.eps, x_out=x, out_scale=self.geo.logit_scale)
        logits = self.lm_head(h)
        return softcap_(logits, self.geo.logit_softcap) if self.geo.logit_softcap else logits

    # --------------------------------------------------------------------------------- #
    # synthetic weights (benchmarks, tests): seeded, every tensor in a range that keeps the stack well-conditioned
    # --------------------------------------------------------------------------------- #
    @torch.no_grad()
    def init_synthetic(self, seed: int = 0, device="cuda") -> "LayeredLM":
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        self.to(device)

        def fill(p, std=None, mean=0.0, lo=None, hi=None):
            if lo is not None:
                v = torch.rand(p.shape, generator=g) * (hi - lo) + lo
            else:
                v = torch.randn(p.shape, generator=g) * std + mean
            p.data.copy_(v.to(p.dtype))

        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if name.endswith("proj.weight") or name.endswith("lm_head.weight"):
                fill(p, std=1.0 / (p.shape[1] ** 0.5))
            elif name in ("embed_tokens.weight", "pair_table"):
                fill(p, std=1.0)
            elif leaf in ("norm1_weight", "norm2_weight", "norm_weight", "q_norm_weight", "k_norm_weight", "out_norm_weight",
                          "norm1b_weight", "norm2b_weight", "kv_norm_weight", "ssd_norm_weight"):
                fill(p, std=0.1, mean=1.0)
            elif leaf in ("uk_weight", "uv_weight", "router_weight", "gate_up_weight", "down_weight", "shared_scale_weight"):
                fill(p, std=1.0 / (p.shape[-1] ** 0.5))
            elif leaf in ("rg1_bias", "rg2_bias", "z_bias", "x_bias", "qkv_bias", "conv_bias", "down_bias", "decay_bias", "dt_bias") \
                    or name.endswith("proj.bias"):
                fill(p, std=0.5)
            elif leaf in ("a_log", "skip"):
                fill(p, lo=-1.0, hi=1.0)
            elif leaf == "correction":
                fill(p, std=0.02)
            elif leaf == "conv_weight":
                fill(p, std=p.shape[1] ** -0.5)
            elif leaf == "value_blend":
                fill(p, lo=0.2, hi=0.6)
            elif leaf in ("shift", "lower"):
                fill(p, lo=0.0, hi=0.9)
            elif leaf in ("f_bias", "sink", "act", "loop_step"):
                fill(p, std=0.5)
            else:
                raise RuntimeError(f"init_synthetic: no rule for {name}")
        return self
