"""Engine configuration: model architecture presets + the serving flags.

The CLI surface mirrors what the reference's Helm chart renders for an engine container
(/root/reference/helm/templates/deployment-vllm-multi.yaml:108-199) and the LMCACHE_* env
contract (same file :256-344), so an unmodified values.yaml drives this engine.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

import torch


@dataclass(frozen=True)
class LatentMixerSpec:
    """A latent-attention mixer: queries and keys/values pass through low-rank latents; a head's
    query/key has ``dim`` unrotated and ``rot_dim`` rotated channels (the rotated key part is one
    vector shared by all heads), its value ``vdim`` channels.  Only the KV latent (``kv_rank``) and
    the rotated key part are cached.  ``kv_from``: the layer whose cache entries this layer reads
    instead of writing its own (it then has no KV down-projection)."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    rope_base: float
    rope_dims: int
    scale: float
    kv_from: int | None = None
    sink: bool = True          # a learned per-head logit in the softmax denominator
    out_gate: bool = True      # head outputs times sigmoid(W_g h)

    @property
    def entry(self) -> int:    # cached values per token
        return self.kv_rank + self.rot_dim

    def weight_count(self, width: int) -> int:
        n = width * (self.q_rank + self.heads) + self.q_rank * self.heads * (self.dim + self.rot_dim)
        n += self.heads * self.vdim * width + self.heads * self.kv_rank * (self.dim + self.vdim)
        return n + (width * self.entry if self.kv_from is None else 0)


@dataclass(frozen=True)
class FeedForwardSpec:
    """``dense``: down(act(up x)), act = relu(.)^2 unless ``act`` says otherwise.  ``moe``: ``experts`` clamped gated units of width ``ff``, ``top``
    per token out of the ``keep`` best of ``groups`` groups, sigmoid scores times ``route_scale``;
    an always-on shared unit of width ``shared_ff`` (0 = none) with a per-token sigmoid gate."""
    kind: str = "dense"
    ff: int = 0
    act: str = "relu_sq"       # relu_sq | xielu (two learned curvatures, see ops.xielu) | gelu_tanh | silu (gated units)
    gated: bool = False        # down(act(gate x) * (up x)) instead of down(act(up x))
    router: str = "sigmoid"    # sigmoid: as described above | softmax: softmax scores, a learned selection bias,
                               # a group scores its largest biased score, weights = scores, not renormalised
    identity: int = 0          # softmax router: extra outputs whose "expert" returns the token itself
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    route_scale: float = 1.0
    norm_topk: bool = False    # sigmoid router: the chosen scores are divided by their sum (+ 1e-20) first
    limit: float = 0.0
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclass(frozen=True)
class LayerSpec:
    type: str
    mixer: LatentMixerSpec
    mlp: FeedForwardSpec | None = None


@dataclass(frozen=True)
class RotarySpec:
    """Rotary positions on the first ``dims`` channels of a head.  ``layout``: which channels form a
    pair, ``half`` = (i, i + dims / 2), ``pairs`` = (2 i, 2 i + 1).  ``scaling`` = (factor, original,
    fast, slow): frequencies whose wavelength exceeds the original context are divided by ``factor``
    behind a linear ramp between the channels that make ``fast`` and ``slow`` turns over it, and cos
    and sin carry the factor 0.1 ln(factor) + 1."""
    base: float
    dims: int
    layout: str = "half"
    scaling: tuple | None = None
    linear: float | None = None   # every frequency divided by this factor (position interpolation)

    def table_scaling(self) -> dict | None:
        if self.linear is not None:
            return {"rope_type": "linear", "factor": self.linear}
        if self.scaling is None:
            return None
        factor, original, fast, slow = self.scaling
        return {"rope_type": "ramp", "factor": factor, "original": original, "fast": fast, "slow": slow}


@dataclass(frozen=True)
class RetentionSpec:
    """Un-normalised linear attention, one constant decay for each head: per head a
    ``dim`` x ``vdim`` state S <- decay S + k v^T, read by the rotated query; head outputs are brought
    to unit root mean square and gated by silu(W_g h)."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: RotarySpec

    def state_elems(self) -> int:
        return self.heads * self.dim * self.vdim

    def weight_count(self, width: int) -> int:
        return width * self.heads * (2 * self.dim + 2 * self.vdim) + self.heads * self.vdim * width

    def token_flops(self) -> float:      # the state update and its read-out, per token
        return 4.0 * self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Grouped-query softmax attention behind a short causal convolution of q, k and v: capped scores
    (cap tanh(s / cap)), a sliding window of ``window`` positions that also keeps the first
    ``keep_first`` tokens, a per-head sink logit in the denominator, and the heads' weights mixed by
    an [heads, heads] matrix after the softmax."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    window: int
    keep_first: int
    rot: RotarySpec
    scale: float
    softcap: float

    @property
    def channels(self) -> int:           # of the fused q | k | v projection
        return self.heads * self.dim + self.kv_heads * (self.dim + self.vdim)

    def state_elems(self) -> int:        # the projected rows the convolution still needs
        return max(self.conv - 1, 0) * self.channels

    def cache_elems(self) -> int:        # per token: rotated keys and values of every KV head
        return self.kv_heads * (self.dim + self.vdim)

    def weight_count(self, width: int) -> int:
        return width * self.channels + self.heads * self.vdim * width


@dataclass(frozen=True)
class GatedRecurrenceSpec:
    """Linear attention with the input gate tied to the forget gate: S <- diag(f) S + (1 - f) v^T,
    f = lower + (1 - lower) sigmoid(W_f h + b) per head and query channel; q = silu(W_q h); head
    outputs are RMS-normed with one weight vector shared by the heads."""
    heads: int
    dim: int
    vdim: int

    def state_elems(self) -> int:
        return self.heads * self.dim * self.vdim

    def weight_count(self, width: int) -> int:
        return width * self.heads * (2 * self.dim + self.vdim) + self.heads * self.vdim * width

    def token_flops(self) -> float:
        return 4.0 * self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers that read the same input; the layer adds left_scale * left + right_scale * right.  ``normed``:
    each output is first RMS-normed over the model width with a weight vector of its own."""
    left: object
    right: object
    left_scale: float
    right_scale: float
    normed: bool = False

    def weight_count(self, width: int) -> int:
        return self.left.weight_count(width) + self.right.weight_count(width)


@dataclass(frozen=True)
class DiffAttentionSpec:
    """Differential grouped-query attention: every head has two query / key maps over the same values,
    o = a1 - lambda a2 with one learned lambda per layer (exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff``), brought to
    unit RMS per head and multiplied by 1 - ``diff``.  q and k are RMS-normed per head and map (one weight vector
    each), rotary positions on their first ``rot.dims`` channels; ``chunk`` > 0: a position sees the keys of its own
    chunk of that many positions (counted from 0) up to itself, 0: plain causal."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    diff: float
    rot: RotarySpec
    chunk: int
    scale: float

    def cache_elems(self) -> int:        # per token: both key maps and the values of every KV head
        return self.kv_heads * (2 * self.dim + self.vdim)

    def weight_count(self, width: int) -> int:
        return width * (2 * self.heads * self.dim + self.kv_heads * (2 * self.dim + self.vdim)) + self.heads * self.vdim * width

    def token_flops(self) -> float:      # a bound: both maps over a full chunk (a quarter of a 32k context without one)
        return 4.0 * self.heads * (self.dim + self.vdim) * (self.chunk or 8192)


@dataclass(frozen=True)
class PooledWindowSpec:
    """Grouped-query softmax attention over a sliding window of ``window`` positions and, in the same softmax, one
    mean key / mean value per block of ``pool`` tokens that lies wholly before the window (0: none).  q and k are
    RMS-normed per head (one weight vector each), rotary positions on their first ``rot.dims`` channels."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    pool: int
    rot: RotarySpec
    scale: float

    def cache_elems(self) -> int:        # per token: keys and values, and as much again for the pooled entries
        return self.kv_heads * (self.dim + self.vdim) * (2 if self.pool else 1)

    def weight_count(self, width: int) -> int:
        return width * (self.heads * self.dim + self.kv_heads * (self.dim + self.vdim)) + self.heads * self.vdim * width

    def token_flops(self) -> float:      # the window, and the blocks of a context of 16 windows
        keys = min(self.window, 32768) * (1 + (16 // self.pool if self.pool else 0))
        return 2.0 * self.heads * (self.dim + self.vdim) * keys


@dataclass(frozen=True)
class LightningSpec:
    """Linear attention with one fixed decay per head on silu'd projections: S <- decay S + k v^T, o = S^T q with
    q, k, v = silu(W h); the heads side by side are RMS-normed together (one weight vector), gated by sigmoid(W_g h)."""
    heads: int
    dim: int
    vdim: int
    decay: tuple

    def state_elems(self) -> int:
        return self.heads * self.dim * self.vdim

    def weight_count(self, width: int) -> int:
        return width * self.heads * (2 * self.dim + 2 * self.vdim) + self.heads * self.vdim * width

    def token_flops(self) -> float:
        return 4.0 * self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class NormedAttentionSpec:
    """Grouped-query softmax attention without rotation: q and k heads are divided by their root mean
    square (no weight), q grows with the position by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1),
    a per-head sink logit joins the denominator, head outputs are gated by sigmoid(W_g h).  ``kv_from``:
    the layer whose cached keys and values this layer reads instead of projecting its own."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float = 0.0
    temp_every: float = 1.0
    kv_from: int | None = None

    def cache_elems(self) -> int:        # per token, for layers that own their entries
        return self.kv_heads * (self.dim + self.vdim) if self.kv_from is None else 0

    def weight_count(self, width: int) -> int:
        n = width * self.heads * (self.dim + self.vdim) + self.heads * self.vdim * width
        return n + (width * self.kv_heads * (self.dim + self.vdim) if self.kv_from is None else 0)


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A matrix memory with exponential gates: per head S <- exp(f + m' - m) S + exp(i - m) k v^T with a running
    maximum m of the log gates, a normaliser n updated like S with k alone, o = S^T q / (max(|n . q|, exp(-m)) + 1e-6);
    log gates i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)); heads brought to unit RMS, weighted
    and gated by sigmoid(W_g h)."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def weight_count(self, width: int) -> int:
        return width * self.heads * (2 * self.dim + 2 * self.vdim + 2) + self.heads * self.vdim * width

    def token_flops(self) -> float:
        return 4.0 * self.heads * self.dim * (self.vdim + 1)


@dataclass(frozen=True)
class GatedLinearSpec:
    """Linear attention with a decay per key channel: S <- diag(a) S + k v^T, a = sigmoid(W_a2 W_a1 h + b)^(1 / tau)
    through a low-rank pair of projections (``decay_rank``; a checkpoint's tensors decide it); heads RMS-normed
    with one weight vector and gated by silu(W_g h)."""
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = 16

    def weight_count(self, width: int) -> int:
        n = width * self.heads * (2 * self.dim + 2 * self.vdim) + self.heads * self.vdim * width
        return n + self.decay_rank * (width + self.heads * self.dim)

    def token_flops(self) -> float:
        return 4.0 * self.heads * self.dim * self.vdim


def pelatar_layers(layers: list[dict]) -> tuple:
    """The ``layers`` list of a Pelatar config.json -> layer specs."""
    out = []
    for i, entry in enumerate(layers):
        m = entry["mixer"]
        kind = entry["type"]
        if kind == "attention":
            temp = m.get("q_temp") or {}
            src = m.get("kv_from")
            mixer = NormedAttentionSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]), temp_coef=float(temp.get("coef", 0.0)), temp_every=float(temp.get("every", 1.0)),
                kv_from=None if src is None else int(src))
            if mixer.heads % mixer.kv_heads or (mixer.temp_coef != 0.0 and mixer.temp_every <= 0):
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads and the temperature's period positive")
            if mixer.kv_from is not None:
                if not 0 <= mixer.kv_from < i:
                    raise ValueError(f"layer {i}: kv_from must name an earlier layer")
                s = out[mixer.kv_from].mixer
                if (not isinstance(s, NormedAttentionSpec) or s.kv_from is not None
                        or (s.kv_heads, s.dim, s.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim)):
                    raise ValueError(f"layer {i}: layer {mixer.kv_from} does not hold keys and values of this layer's shape")
        elif kind == "mlstm":
            mixer = MatrixMemorySpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]))
            if mixer.gate_cap <= 0:
                raise ValueError(f"layer {i}: gate_cap must be positive")
        elif kind == "gla":
            mixer = GatedLinearSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]),
                                    int(m.get("decay_rank", 16)))
            if mixer.tau <= 0:
                raise ValueError(f"layer {i}: tau must be positive")
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = entry.get("mlp")
        mlp = None
        if f is not None:
            if f["kind"] == "dense":
                mlp = FeedForwardSpec(kind="dense", ff=int(f["ff"]), act="gelu_tanh", gated=True)
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                ident = int(r.get("identity", 0))
                mlp = FeedForwardSpec(kind="moe", ff=int(f["expert"]["ff"]), act="silu", gated=True, experts=int(r["experts"]),
                                      top=int(r["top"]), groups=int(g.get("count", 1)),
                                      keep=int(g.get("keep", g.get("count", 1))), router="softmax", identity=ident)
                n = mlp.experts + ident
                if mlp.groups < 1 or n % mlp.groups or not 1 <= mlp.keep <= mlp.groups or mlp.top > n // mlp.groups * mlp.keep:
                    raise ValueError(f"layer {i}: experts and identity experts must split into equal groups that hold `top`")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        out.append(LayerSpec(kind, mixer, mlp))
    return tuple(out)


def pelatar_config(name: str, vocab: int, width: int, layers: list[dict], norm_eps: float = 1e-5,
                   max_position_embeddings: int = 32768) -> "ModelConfig":
    specs = pelatar_layers(layers)
    att = [s.mixer for s in specs if isinstance(s.mixer, NormedAttentionSpec)]
    return ModelConfig(
        name=name, architecture="pelatar", vocab_size=int(vocab), hidden_size=int(width),
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] + [0]), num_layers=len(specs),
        num_heads=max(s.mixer.heads for s in specs), num_kv_heads=max([a.kv_heads for a in att] + [1]),
        head_dim=max(s.mixer.dim for s in specs), norm_eps=float(norm_eps),
        max_position_embeddings=max_position_embeddings, tie_word_embeddings=True, layer_specs=specs,
        bos_token_id=0, eos_token_id=-1)  # the design names no special tokens


def _positive(i: int, **values) -> None:
    for k, v in values.items():
        if v < 1:
            raise ValueError(f"layer {i}: {k} must be at least 1")


def zetalorn_layers(layers: list[dict]) -> tuple:
    """The ``layers`` list of a Zetalorn config.json -> layer specs."""

    def rotary(rot: dict | None, layout: str, dim: int, i: int) -> RotarySpec:
        rot = rot or {"base": 10000.0, "dims": 0}
        sc = rot.get("scaling")
        spec = RotarySpec(float(rot["base"]), int(rot["dims"]), layout, None, float(sc["factor"]) if sc else None)
        if spec.dims % 2 or not 0 <= spec.dims <= dim or (spec.linear is not None and spec.linear <= 0):
            raise ValueError(f"layer {i}: rotary dims must be even and within the head, a scaling factor positive")
        return spec

    out = []
    for i, entry in enumerate(layers):
        m = entry["mixer"]
        kind = entry["type"]
        if kind == "attention":
            mask = m.get("mask") or {}
            mixer = DiffAttentionSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                diff=float(m["diff"]), rot=rotary(m.get("rot"), "pairs", int(m["dim"]), i), chunk=int(mask.get("size", 0)),
                scale=float(m["scale"]))
            _positive(i, heads=mixer.heads, kv_heads=mixer.kv_heads, dim=mixer.dim, vdim=mixer.vdim)
            if mixer.heads % mixer.kv_heads or mixer.chunk < 0:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads and the chunk size positive")
        elif kind == "parallel":
            a, r = m["left"], m["right"]
            mask = a.get("mask") or {}
            left = PooledWindowSpec(
                heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                window=int(mask.get("size", 1 << 30)), pool=int(mask.get("pool", 0)),
                rot=rotary(a.get("rot"), "half", int(a["dim"]), i), scale=float(a["scale"]))
            _positive(i, heads=left.heads, kv_heads=left.kv_heads, dim=left.dim, vdim=left.vdim, window=left.window)
            if left.heads % left.kv_heads or left.pool < 0:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads and the pooled block size positive")
            right = LightningSpec(int(r["heads"]), int(r["dim"]), int(r["vdim"]), tuple(float(d) for d in r["decay"]))
            _positive(i, right_heads=right.heads, right_dim=right.dim, right_vdim=right.vdim)
            if len(right.decay) != right.heads or not all(0.0 <= d <= 1.0 for d in right.decay):
                raise ValueError(f"layer {i}: one decay within [0, 1] per head is required")
            mixer = ParallelMixerSpec(left, right, 0.5, 0.5, normed=True)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = entry.get("mlp")
        mlp = None
        if f is not None:
            if f.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
            r, ex = f["router"], f["expert"]
            g = r.get("groups") or {}
            mlp = FeedForwardSpec(
                kind="moe", ff=int(ex["ff"]), gated=True, experts=int(r["experts"]), top=int(r["top"]),
                groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))), norm_topk=True,
                limit=float(ex["limit"]))
            if (mlp.groups < 1 or mlp.experts % mlp.groups or not 1 <= mlp.keep <= mlp.groups
                    or not 1 <= mlp.top <= mlp.experts // mlp.groups * mlp.keep or mlp.ff < 1):
                raise ValueError(f"layer {i}: experts must split into equal groups, and the kept groups hold `top`")
        out.append(LayerSpec(kind, mixer, mlp))
    return tuple(out)


def zetalorn_config(name: str, vocab: int, width: int, layers: list[dict], loop: dict | None = None,
                    logit_scale: float = 1.0, norm_eps: float = 1e-6, max_position_embeddings: int = 32768) -> "ModelConfig":
    specs = zetalorn_layers(layers)
    runs = None
    if loop:
        runs = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
        if not 0 <= runs[0] < runs[1] <= len(specs) or runs[2] < 1:
            raise ValueError("loop: 0 <= start < stop <= layers and times >= 1 are required")
    att = [s.mixer.left if s.type == "parallel" else s.mixer for s in specs]
    return ModelConfig(
        name=name, architecture="zetalorn", vocab_size=int(vocab), hidden_size=int(width),
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] + [0]), num_layers=len(specs),
        num_heads=max(a.heads for a in att), num_kv_heads=max(a.kv_heads for a in att),
        head_dim=max(a.dim for a in att), norm_eps=float(norm_eps), max_position_embeddings=max_position_embeddings,
        tie_word_embeddings=False, logit_scale=float(logit_scale), layer_specs=specs, layer_loop=runs,
        bos_token_id=0, eos_token_id=-1)  # the design names no special tokens


def _rotary(rot: dict, layout: str) -> RotarySpec:
    sc = rot.get("scaling")
    scaling = None if not sc else (float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))
    dims = int(rot["dims"])
    if dims % 2:
        raise ValueError("rotary dims must be even")
    return RotarySpec(float(rot["base"]), dims, layout, scaling)


def revelix_layers(layers: list[dict]) -> tuple:
    """The ``layers`` list of a Revelix config.json -> layer specs."""
    out = []
    for i, entry in enumerate(layers):
        m = entry["mixer"]
        kind = entry["type"]
        if kind == "retention":
            mixer = RetentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), tuple(float(d) for d in m["decay"]),
                                  _rotary(m["rot"], "half"))
            if len(mixer.decay) != mixer.heads or mixer.rot.dims > mixer.dim:
                raise ValueError(f"layer {i}: one decay per head and rotary dims within the head are required")
        elif kind == "parallel":
            a, r = m["left"], m["right"]
            left = WindowAttentionSpec(
                heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                conv=int(a["conv"]), window=int(a["mask"]["size"]), keep_first=int(a["mask"]["keep_first"]),
                rot=_rotary(a["rot"], "pairs"), scale=float(a["scale"]), softcap=float(a["softcap"]))
            if left.heads % left.kv_heads or left.conv < 1 or left.window < 1 or left.rot.dims > left.dim:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, conv and window at least 1, "
                                 "rotary dims within the head")
            right = GatedRecurrenceSpec(int(r["heads"]), int(r["dim"]), int(r["vdim"]))
            mixer = ParallelMixerSpec(left, right, float(m["left_scale"]), float(m["right_scale"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        f = entry.get("mlp")
        mlp = None
        if f is not None:
            if f["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
            mlp = FeedForwardSpec(kind="dense", ff=int(f["ff"]), act="xielu")
        out.append(LayerSpec(kind, mixer, mlp))
    return tuple(out)


def revelix_config(name: str, vocab: int, width: int, layers: list[dict], logit_scale: float = 1.0,
                   norm_eps: float = 1e-6, max_position_embeddings: int = 32768) -> "ModelConfig":
    specs = revelix_layers(layers)
    heads = [s.mixer.left.heads if s.type == "parallel" else s.mixer.heads for s in specs]
    dims = [s.mixer.left.dim if s.type == "parallel" else s.mixer.dim for s in specs]
    return ModelConfig(
        name=name, architecture="revelix", vocab_size=int(vocab), hidden_size=int(width),
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] + [0]), num_layers=len(specs),
        num_heads=max(heads), num_kv_heads=max([s.mixer.left.kv_heads for s in specs if s.type == "parallel"] + [1]),
        head_dim=max(dims), norm_eps=float(norm_eps), max_position_embeddings=max_position_embeddings,
        tie_word_embeddings=True, logit_scale=float(logit_scale), layer_specs=specs,
        bos_token_id=0, eos_token_id=-1)  # the design names no special tokens


def zururax_layers(layers: list[dict]) -> tuple:
    """The ``layers`` list of a Zururax config.json -> layer specs."""
    out = []
    for i, entry in enumerate(layers):
        if entry["type"] != "latent_attention":
            raise ValueError(f"layer {i}: unknown mixer type {entry['type']!r}")
        m = entry["mixer"]
        rot = m.get("rot") or {}
        src = m.get("kv_from")
        mixer = LatentMixerSpec(
            heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
            kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), rope_base=float(rot.get("base", 10000.0)),
            rope_dims=int(rot.get("dims", m["rot_dim"])), scale=float(m["scale"]),
            kv_from=None if src is None else int(src))
        if mixer.kv_from is not None:
            if not 0 <= mixer.kv_from < i:
                raise ValueError(f"layer {i}: kv_from must name an earlier layer")
            s = out[mixer.kv_from].mixer
            if s.kv_from is not None or (s.kv_rank, s.rot_dim) != (mixer.kv_rank, mixer.rot_dim):
                raise ValueError(f"layer {i}: layer {mixer.kv_from} does not hold entries of this layer's shape")
        f = entry.get("mlp")
        mlp = None
        if f is not None:
            if f["kind"] == "dense":
                mlp = FeedForwardSpec(kind="dense", ff=int(f["ff"]))
            elif f["kind"] == "moe":
                r, ex, sh = f["router"], f["expert"], f.get("shared")
                g = r.get("groups") or {}
                mlp = FeedForwardSpec(
                    kind="moe", ff=int(ex["ff"]), experts=int(r["experts"]), top=int(r["top"]),
                    groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))),
                    route_scale=float(r.get("scale", 1.0)), limit=float(ex["limit"]),
                    shared_ff=int(sh["ff"]) if sh else 0, shared_limit=float(sh["limit"]) if sh else 0.0)
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        out.append(LayerSpec("latent_attention", mixer, mlp))
    return tuple(out)


def zururax_config(name: str, vocab: int, width: int, layers: list[dict], embedding_scale: float = 1.0,
                   norm_eps: float = 1e-5, max_position_embeddings: int = 8192) -> "ModelConfig":
    specs = zururax_layers(layers)
    return ModelConfig(
        name=name, architecture="zururax", vocab_size=int(vocab), hidden_size=int(width),
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] + [0]), num_layers=len(specs),
        num_heads=max(s.mixer.heads for s in specs), num_kv_heads=1,
        head_dim=max(s.mixer.dim + s.mixer.rot_dim for s in specs), norm_eps=float(norm_eps),
        max_position_embeddings=max_position_embeddings, embedding_scale=float(embedding_scale),
        layer_specs=specs, bos_token_id=0, eos_token_id=-1)  # the design names no special tokens


@dataclass
class ModelConfig:
    name: str = "tiny-llama"
    architecture: str = "llama"  # llama | mixtral | opt | gpt2 | zururax | revelix | pelatar | zetalorn
    vocab_size: int = 512
    hidden_size: int = 256
    intermediate_size: int = 512
    num_layers: int = 2
    num_heads: int = 2
    num_kv_heads: int = 1
    head_dim: int = 128
    rope_theta: float = 10000.0
    rope_scaling: dict | None = None
    norm_eps: float = 1e-5
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    num_experts: int = 0
    num_experts_per_tok: int = 0
    qkv_bias: bool = False  # Qwen2 family, Llama-style checkpoints with attention_bias
    bos_token_id: int = 1
    eos_token_id: int = 2
    extra_eos_token_ids: tuple = ()  # config.json may list several end-of-sequence ids
    # OPT / GPT-2 specifics (learned positions, LayerNorm, biased projections)
    ffn_dim: int = 0
    pos_offset: int = 0
    activation: str = "relu"  # relu (OPT) | gelu_new (GPT-2)
    # designs whose layers differ from one another list them (Zururax); empty = num_layers equal layers
    layer_specs: tuple = ()
    embedding_scale: float = 1.0
    logit_scale: float = 1.0   # logits = head(x) * logit_scale
    # (start, stop, times): layers start .. stop - 1 run `times` times in a row with the same weights, every pass
    # with cache entries and state of its own
    layer_loop: tuple | None = None

    def layer_runs(self) -> list:
        """(layer index, pass number when the run starts a pass of the loop, else None) of every layer run."""
        n = len(self.layer_specs)
        if not self.layer_loop:
            return [(i, None) for i in range(n)]
        start, stop, times = self.layer_loop
        runs = [(i, None) for i in range(start)]
        for t in range(times):
            runs += [(i, t if i == start else None) for i in range(start, stop)]
        return runs + [(i, None) for i in range(stop, n)]

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def prefill_flops(self) -> tuple[float, float]:
        """(GEMM FLOPs per new token, attention FLOPs per (new token x context token) pair)."""
        h, i = self.hidden_size, self.intermediate_size
        if self.layer_specs:
            gemm = pair = 0.0
            for s in [self.layer_specs[i] for i, _ in self.layer_runs()]:
                m, f = s.mixer, s.mlp
                gemm += m.weight_count(h)
                if isinstance(m, LatentMixerSpec):
                    pair += m.heads * (m.entry + m.kv_rank)
                elif isinstance(m, NormedAttentionSpec):
                    pair += m.heads * (m.dim + m.vdim)
                else:  # recurrences cost per token, a windowed softmax at most its window per token
                    for part in (getattr(m, "left", None), getattr(m, "right", None), m):
                        if hasattr(part, "token_flops"):
                            gemm += part.token_flops() / 2.0
                        if isinstance(part, WindowAttentionSpec):
                            gemm += part.heads * (part.dim + part.kv_heads * part.vdim) * (part.window + part.keep_first)
                if f is not None:
                    gemm += ((3 if f.gated else 2) * h * f.ff if f.kind == "dense"
                             else 3 * h * (f.top * f.ff + f.shared_ff) + h * (f.experts + f.identity))
            return 2.0 * gemm, 2.0 * pair
        attn_w = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        mlp_w = 3 * h * i * max(1, self.num_experts_per_tok if self.num_experts else 1)
        return 2.0 * self.num_layers * (attn_w + mlp_w), 4.0 * self.num_layers * self.q_size

    def num_params(self) -> int:
        h, i, l_ = self.hidden_size, self.intermediate_size, self.num_layers
        if self.layer_specs:
            n = self.vocab_size * h * (1 if self.tie_word_embeddings else 2)
            for s in self.layer_specs:
                m, f = s.mixer, s.mlp
                n += m.weight_count(h)
                if f is not None:
                    n += ((3 if f.gated else 2) * h * f.ff if f.kind == "dense"
                          else 3 * h * (f.experts * f.ff + f.shared_ff) + h * (f.experts + f.identity))
            return n
        attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        mlp = 3 * h * i * max(1, self.num_experts)
        emb = self.vocab_size * h * (1 if self.tie_word_embeddings else 2)
        return l_ * (attn + mlp) + emb


PRESETS: dict[str, ModelConfig] = {
    "llama-3-8b": ModelConfig(
        name="llama-3-8b", architecture="llama", vocab_size=128256, hidden_size=4096,
        intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128,
        rope_theta=500000.0, norm_eps=1e-5, max_position_embeddings=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        bos_token_id=128000, eos_token_id=128009),
    "mixtral-8x7b": ModelConfig(
        name="mixtral-8x7b", architecture="mixtral", vocab_size=32000, hidden_size=4096,
        intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128,
        rope_theta=1000000.0, norm_eps=1e-5, max_position_embeddings=32768, num_experts=8,
        num_experts_per_tok=2, bos_token_id=1, eos_token_id=2),
    "opt-125m": ModelConfig(
        name="opt-125m", architecture="opt", vocab_size=50272, hidden_size=768,
        intermediate_size=3072, num_layers=12, num_heads=12, num_kv_heads=12, head_dim=64,
        max_position_embeddings=2048, ffn_dim=3072, pos_offset=2, tie_word_embeddings=True,
        bos_token_id=2, eos_token_id=2),
    # the other models the reference's tutorials and CI values name
    "mistral-7b": ModelConfig(
        name="mistral-7b", architecture="llama", vocab_size=32000, hidden_size=4096,
        intermediate_size=14336, num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128,
        rope_theta=1000000.0, norm_eps=1e-5, max_position_embeddings=32768, bos_token_id=1, eos_token_id=2),
    "llama-3-70b": ModelConfig(
        name="llama-3-70b", architecture="llama", vocab_size=128256, hidden_size=8192,
        intermediate_size=28672, num_layers=80, num_heads=64, num_kv_heads=8, head_dim=128,
        rope_theta=500000.0, norm_eps=1e-5, max_position_embeddings=131072,
        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        bos_token_id=128000, eos_token_id=128009),
    "llama-3.2-1b": ModelConfig(
        name="llama-3.2-1b", architecture="llama", vocab_size=128256, hidden_size=2048,
        intermediate_size=8192, num_layers=16, num_heads=32, num_kv_heads=8, head_dim=64,
        rope_theta=500000.0, norm_eps=1e-5, max_position_embeddings=131072, tie_word_embeddings=True,
        rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        bos_token_id=128000, eos_token_id=128009),
    "smollm2-135m": ModelConfig(
        name="smollm2-135m", architecture="llama", vocab_size=49152, hidden_size=576,
        intermediate_size=1536, num_layers=30, num_heads=9, num_kv_heads=3, head_dim=64,
        rope_theta=100000.0, norm_eps=1e-5, max_position_embeddings=8192, tie_word_embeddings=True,
        bos_token_id=1, eos_token_id=2),
    "distilgpt2": ModelConfig(
        name="distilgpt2", architecture="gpt2", vocab_size=50257, hidden_size=768,
        intermediate_size=3072, num_layers=6, num_heads=12, num_kv_heads=12, head_dim=64,
        max_position_embeddings=1024, ffn_dim=3072, pos_offset=0, tie_word_embeddings=True,
        activation="gelu_new", bos_token_id=50256, eos_token_id=50256),
    "gpt2": ModelConfig(
        name="gpt2", architecture="gpt2", vocab_size=50257, hidden_size=768,
        intermediate_size=3072, num_layers=12, num_heads=12, num_kv_heads=12, head_dim=64,
        max_position_embeddings=1024, ffn_dim=3072, pos_offset=0, tie_word_embeddings=True,
        activation="gelu_new", bos_token_id=50256, eos_token_id=50256),
    "tiny-gpt2": ModelConfig(name="tiny-gpt2", architecture="gpt2", vocab_size=512, hidden_size=128,
                             intermediate_size=256, ffn_dim=256, num_layers=2, num_heads=4,
                             num_kv_heads=4, head_dim=32, pos_offset=0, tie_word_embeddings=True,
                             activation="gelu_new", max_position_embeddings=2048),
    "tiny-llama": ModelConfig(name="tiny-llama"),
    "tiny-llama-gqa": ModelConfig(name="tiny-llama-gqa", num_heads=8, num_kv_heads=2,
                                  hidden_size=512, intermediate_size=1024, num_layers=3),
    # Qwen2 family: biased q/k/v projections, GQA group of 7 on the 7B model
    "qwen2.5-7b": ModelConfig(
        name="qwen2.5-7b", architecture="llama", vocab_size=152064, hidden_size=3584,
        intermediate_size=18944, num_layers=28, num_heads=28, num_kv_heads=4, head_dim=128,
        rope_theta=1000000.0, norm_eps=1e-6, max_position_embeddings=32768, qkv_bias=True,
        bos_token_id=151643, eos_token_id=151645),
    "tiny-qwen2": ModelConfig(name="tiny-qwen2", num_heads=7, num_kv_heads=1, hidden_size=512,
                              intermediate_size=1024, num_layers=3, qkv_bias=True, norm_eps=1e-6),
    # three query heads per KV head (Llama-3.2-3B's ratio), 128-channel heads
    "tiny-llama-gqa3": ModelConfig(name="tiny-llama-gqa3", num_heads=6, num_kv_heads=2, hidden_size=768,
                                   intermediate_size=1024, num_layers=3),
    "tiny-mixtral": ModelConfig(name="tiny-mixtral", architecture="mixtral", num_heads=4,
                                num_kv_heads=2, hidden_size=256, intermediate_size=256,
                                num_experts=4, num_experts_per_tok=2),
    # expert widths the matrix-core decode kernels tile (whole and halved)
    "tiny-mixtral-wide": ModelConfig(name="tiny-mixtral-wide", architecture="mixtral", num_heads=4,
                                     num_kv_heads=2, hidden_size=256, intermediate_size=1024,
                                     num_experts=4, num_experts_per_tok=2),
    # heads of 64 channels (the geometry of OPT-125m, GPT-2, Llama-3.2-1B, Qwen2-0.5B)
    "tiny-opt-hd64": ModelConfig(name="tiny-opt-hd64", architecture="opt", vocab_size=512, hidden_size=256,
                                 intermediate_size=512, ffn_dim=512, num_layers=2, num_heads=4,
                                 num_kv_heads=4, head_dim=64, pos_offset=2, tie_word_embeddings=True,
                                 max_position_embeddings=2048),
    "tiny-llama-hd64": ModelConfig(name="tiny-llama-hd64", num_heads=8, num_kv_heads=2, head_dim=64,
                                   hidden_size=512, intermediate_size=1024, num_layers=3),
    "tiny-opt": ModelConfig(name="tiny-opt", architecture="opt", vocab_size=512, hidden_size=128,
                            intermediate_size=256, ffn_dim=256, num_layers=2, num_heads=4,
                            num_kv_heads=4, head_dim=32, pos_offset=2, tie_word_embeddings=True,
                            max_position_embeddings=2048),
}



def _zx_mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _zx_moe(ff, experts, top, groups, keep, shared_ff, scale=1.0, limit=7.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}, "scale": scale},
            "shared": {"ff": shared_ff, "limit": limit} if shared_ff else None}


def _zx_layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


# Zururax at random weights: a small one for tests and smoke runs, and one with the layer shapes of a
# mid-sized latent-attention mixture model (benchmarks; every second layer reads its neighbour's cache)
PRESETS["tiny-zururax"] = zururax_config(
    "tiny-zururax", 512, 192,
    [_zx_layer(_zx_mixer(3, 16, 8, 24, 48, 40), {"kind": "dense", "ff": 320}),
     _zx_layer(_zx_mixer(3, 16, 8, 24, 48, 40, kv_from=0), _zx_moe(48, 8, 2, 2, 1, 80, scale=1.5, limit=1.0)),
     _zx_layer(_zx_mixer(2, 24, 16, 16, 64, 56, base=50000.0), _zx_moe(48, 6, 3, 3, 2, 0, scale=2.0, limit=2.0))],
    embedding_scale=2.0, max_position_embeddings=4096)
PRESETS["zururax-bench"] = zururax_config(
    "zururax-bench", 32000, 4096,
    [_zx_layer(_zx_mixer(32, 128, 64, 128, 512, 1536, kv_from=(i - 1 if i % 2 else None)),
               {"kind": "dense", "ff": 14336} if i == 0 else _zx_moe(2048, 32, 4, 8, 4, 2048, scale=2.5))
     for i in range(8)],
    max_position_embeddings=32768)



def _rx_retention(heads, dim, vdim, mlp=None, base=10000.0):
    return {"type": "retention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": dim},
                      "decay": [1 - 2.0 ** (-5 - 3 * i / heads) for i in range(heads)]}}


def _rx_parallel(heads, kv_heads, dim, vdim, window, keep, r_heads, r_dim, r_vdim, mlp=None, conv=4):
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                               "mask": {"size": window, "keep_first": keep},
                               "rot": {"base": 1e6, "dims": dim,
                                       "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                               "scale": dim ** -0.5, "softcap": 50.0},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim},
                      "left_scale": 0.7, "right_scale": 0.7}}


# Revelix at random weights: a small one for smoke runs, and one with layer shapes of a 2048-wide model
PRESETS["tiny-revelix"] = revelix_config(
    "tiny-revelix", 512, 128,
    [_rx_retention(2, 32, 64, {"kind": "dense", "ff": 256}),
     _rx_parallel(4, 2, 64, 64, 96, 2, 2, 32, 64, {"kind": "dense", "ff": 256}),
     _rx_retention(2, 32, 64)], logit_scale=0.5, max_position_embeddings=4096)
PRESETS["revelix-bench"] = revelix_config(
    "revelix-bench", 32000, 2048,
    [_rx_retention(16, 128, 256, {"kind": "dense", "ff": 8192}) if i % 3 == 0 else
     _rx_parallel(16, 4, 128, 128, 1024, 4, 8, 128, 128, {"kind": "dense", "ff": 8192}) for i in range(6)],
    logit_scale=0.5, max_position_embeddings=32768)

def _px_moe(ff, experts, top, groups, keep, identity):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}, "identity": identity}}


def _px_attention(heads, kv_heads, dim, vdim, mlp=None, kv_from=None, every=256):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
         "q_temp": {"coef": 0.4, "every": every}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def pelatar_stack(width, heads, ff, experts, unit_ff, top, identity, blocks=1):
    """Layer list of a Pelatar at random weights: per block a matrix memory, a gated linear attention, an attention
    layer and a second one that reads the first one's keys and values; dense and routed feed-forwards in turn."""
    dense = {"kind": "dense", "ff": ff}
    routed = _px_moe(unit_ff, experts, top, 4, 2, identity)
    out = []
    for b in range(blocks):
        out += [{"type": "mlstm", "mlp": dense, "mixer": {"heads": heads // 2, "dim": 128, "vdim": 256, "gate_cap": 12.0}},
                {"type": "gla", "mlp": routed, "mixer": {"heads": heads // 2, "dim": 128, "vdim": 256, "tau": 8.0}},
                _px_attention(heads, heads // 4, 128, 128, dense),
                _px_attention(heads, heads // 4, 128, 128, routed, kv_from=4 * b + 2)]
    return out


# Pelatar at random weights: a small one for smoke runs, and one with layer shapes of a 2048-wide model
PRESETS["tiny-pelatar"] = pelatar_config(
    "tiny-pelatar", 512, 128,
    [{"type": "mlstm", "mlp": {"kind": "dense", "ff": 256}, "mixer": {"heads": 2, "dim": 32, "vdim": 64, "gate_cap": 12.0}},
     {"type": "gla", "mlp": _px_moe(64, 6, 2, 2, 1, 2), "mixer": {"heads": 2, "dim": 64, "vdim": 32, "tau": 8.0}},
     _px_attention(4, 2, 64, 128, {"kind": "dense", "ff": 256}, every=64),
     _px_attention(4, 2, 64, 128, _px_moe(64, 4, 2, 1, 1, 0), kv_from=2, every=64)], max_position_embeddings=4096)
PRESETS["pelatar-bench"] = pelatar_config("pelatar-bench", 32000, 2048, pelatar_stack(2048, 16, 5632, 28, 1024, 4, 4),
                                          max_position_embeddings=32768)


def _zx_moe(ff, experts, top, groups, keep, limit=7.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def _zx_attention(heads, kv_heads, dim, vdim, chunk, mlp=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": 0.2, "scale": dim ** -0.5,
                      "mask": {"size": chunk}, "rot": {"base": 10000.0, "dims": dim // 2, "scaling": {"factor": 4.0}}}}


def _zx_parallel(heads, kv_heads, dim, vdim, window, pool, r_heads, r_dim, r_vdim, mlp=None):
    decay = [1.0 - 2.0 ** (-5.0 - 3.0 * i / max(r_heads - 1, 1)) for i in range(r_heads)]
    return {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                               "mask": {"size": window, "pool": pool}, "rot": {"base": 50000.0, "dims": dim}},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": decay}}}


def zetalorn_stack(width, heads, experts, unit_ff, top, blocks=1):
    """Layer list of a Zetalorn at random weights: per block a differential attention layer over chunks of 2048
    positions and a parallel layer (a window of 1024 positions with blocks of 16 tokens pooled before it, beside a
    lightning recurrence with half as many heads), both with a routed feed-forward."""
    routed = _zx_moe(unit_ff, experts, top, 4, 2)
    out = []
    for _ in range(blocks):
        out += [_zx_attention(heads, heads // 4, 128, 128, 2048, routed),
                _zx_parallel(heads, heads // 4, 128, 128, 1024, 16, heads // 2, 128, 256, routed)]
    return out


# Zetalorn at random weights: a small one for smoke runs, and one with layer shapes of a 2048-wide model whose
# two layers run twice
PRESETS["tiny-zetalorn"] = zetalorn_config(
    "tiny-zetalorn", 512, 128,
    [_zx_parallel(4, 2, 64, 128, 80, 8, 2, 32, 64, _zx_moe(64, 6, 2, 2, 1)),
     _zx_attention(4, 2, 64, 128, 160, _zx_moe(64, 4, 2, 1, 1)),
     _zx_parallel(2, 1, 64, 128, 64, 16, 2, 64, 32)], loop={"start": 0, "stop": 2, "times": 2}, logit_scale=0.5,
    max_position_embeddings=4096)
PRESETS["zetalorn-bench"] = zetalorn_config("zetalorn-bench", 32000, 2048, zetalorn_stack(2048, 16, 16, 1024, 4),
                                            loop={"start": 0, "stop": 2, "times": 2}, logit_scale=0.5)

_ALIASES = {
    "meta-llama/meta-llama-3-8b": "llama-3-8b",
    "meta-llama/meta-llama-3-8b-instruct": "llama-3-8b",
    "meta-llama/llama-3.1-8b": "llama-3-8b",
    "meta-llama/llama-3.1-8b-instruct": "llama-3-8b",
    "mistralai/mixtral-8x7b-v0.1": "mixtral-8x7b",
    "mistralai/mixtral-8x7b-instruct-v0.1": "mixtral-8x7b",
    "facebook/opt-125m": "opt-125m",
    "qwen/qwen2.5-7b-instruct": "qwen2.5-7b",
    "qwen/qwen2.5-7b": "qwen2.5-7b",
    "qwen/qwen2-7b-instruct": "qwen2.5-7b",
    "mistralai/mistral-7b-instruct-v0.2": "mistral-7b",
    "mistralai/mistral-7b-v0.1": "mistral-7b",
    "meta-llama/llama-3.3-70b-instruct": "llama-3-70b",
    "meta-llama/llama-3.1-70b-instruct": "llama-3-70b",
    "meta-llama/meta-llama-3-70b-instruct": "llama-3-70b",
    "meta-llama/llama-3.2-1b-instruct": "llama-3.2-1b",
    "meta-llama/llama-3.2-1b": "llama-3.2-1b",
    "huggingfacetb/smollm2-135m-instruct": "smollm2-135m",
    "distilbert/distilgpt2": "distilgpt2",
    "openai-community/gpt2": "gpt2",
}


def _from_hf_config(cfg: dict[str, Any], name: str) -> ModelConfig:
    if str(cfg.get("architecture", "")).lower() == "zururax":
        return zururax_config(name, cfg["vocab"], cfg["width"], cfg["layers"],
                              embedding_scale=(cfg.get("embedding") or {}).get("scale", 1.0),
                              norm_eps=(cfg.get("norm") or {}).get("eps", 1e-5),
                              max_position_embeddings=int(cfg.get("max_positions", 32768)))
    if str(cfg.get("architecture", "")).lower() == "revelix":
        return revelix_config(name, cfg["vocab"], cfg["width"], cfg["layers"], logit_scale=cfg.get("logit_scale", 1.0),
                              norm_eps=(cfg.get("norm") or {}).get("eps", 1e-6),
                              max_position_embeddings=int(cfg.get("max_positions", 32768)))
    if str(cfg.get("architecture", "")).lower() == "zetalorn":
        return zetalorn_config(name, cfg["vocab"], cfg["width"], cfg["layers"], loop=cfg.get("loop"),
                               logit_scale=cfg.get("logit_scale", 1.0), norm_eps=(cfg.get("norm") or {}).get("eps", 1e-6),
                               max_position_embeddings=int(cfg.get("max_positions", 32768)))
    if str(cfg.get("architecture", "")).lower() == "pelatar":
        return pelatar_config(name, cfg["vocab"], cfg["width"], cfg["layers"],
                              norm_eps=(cfg.get("norm") or {}).get("eps", 1e-5),
                              max_position_embeddings=int(cfg.get("max_positions", 32768)))
    arch = (cfg.get("architectures") or [""])[0].lower()
    mt = cfg.get("model_type", "").lower()
    if "opt" in (arch + mt):
        h = cfg["hidden_size"]
        return ModelConfig(
            name=name, architecture="opt", vocab_size=cfg["vocab_size"], hidden_size=h,
            intermediate_size=cfg["ffn_dim"], ffn_dim=cfg["ffn_dim"],
            num_layers=cfg["num_hidden_layers"], num_heads=cfg["num_attention_heads"],
            num_kv_heads=cfg["num_attention_heads"], head_dim=h // cfg["num_attention_heads"],
            max_position_embeddings=cfg.get("max_position_embeddings", 2048), pos_offset=2,
            tie_word_embeddings=True, bos_token_id=cfg.get("bos_token_id", 2),
            eos_token_id=cfg.get("eos_token_id", 2))
    if "gpt2" in (arch + mt):
        h = cfg["n_embd"]
        inner = cfg.get("n_inner") or 4 * h
        return ModelConfig(
            name=name, architecture="gpt2", vocab_size=cfg["vocab_size"], hidden_size=h,
            intermediate_size=inner, ffn_dim=inner, num_layers=cfg["n_layer"], num_heads=cfg["n_head"],
            num_kv_heads=cfg["n_head"], head_dim=h // cfg["n_head"],
            max_position_embeddings=cfg.get("n_positions", 1024), pos_offset=0, tie_word_embeddings=True,
            activation="gelu_new", norm_eps=cfg.get("layer_norm_epsilon", 1e-5),
            bos_token_id=cfg.get("bos_token_id", 50256), eos_token_id=cfg.get("eos_token_id", 50256))
    is_moe = "mixtral" in (arch + mt)
    if "qwen2" not in (arch + mt) and (cfg.get("attention_bias") or cfg.get("mlp_bias")):
        raise ValueError(f"{name}: projections with biases are only supported for the Qwen2 family")
    # rotary settings: top-level ``rope_theta`` / ``rope_scaling`` (checkpoints written by
    # transformers 4.x) or one ``rope_parameters`` object (5.x)
    rp = cfg.get("rope_parameters") or {}
    rope_theta = cfg.get("rope_theta", rp.get("rope_theta", 10000.0))
    rope_scaling = cfg.get("rope_scaling")
    if rope_scaling is None and rp.get("rope_type", "default") not in ("default", None):
        rope_scaling = {k: v for k, v in rp.items() if k != "rope_theta"}
    h, nh = cfg["hidden_size"], cfg["num_attention_heads"]
    eos = cfg.get("eos_token_id", 2)
    extra_eos: tuple = ()
    if isinstance(eos, list):
        extra_eos = tuple(int(x) for x in eos[1:])
        eos = eos[0]
    return ModelConfig(
        name=name, architecture="mixtral" if is_moe else "llama", vocab_size=cfg["vocab_size"],
        hidden_size=h, intermediate_size=cfg["intermediate_size"],
        num_layers=cfg["num_hidden_layers"], num_heads=nh,
        num_kv_heads=cfg.get("num_key_value_heads", nh), head_dim=cfg.get("head_dim") or h // nh,
        rope_theta=rope_theta, rope_scaling=rope_scaling,
        norm_eps=cfg.get("rms_norm_eps", 1e-5),
        max_position_embeddings=cfg.get("max_position_embeddings", 8192),
        tie_word_embeddings=cfg.get("tie_word_embeddings", False),
        num_experts=cfg.get("num_local_experts", 0),
        num_experts_per_tok=cfg.get("num_experts_per_tok", 0),
        qkv_bias="qwen2" in (arch + mt),
        bos_token_id=cfg.get("bos_token_id") or 1, eos_token_id=eos, extra_eos_token_ids=extra_eos)


def resolve_model(model: str) -> tuple[ModelConfig, Path | None]:
    """Model id or local directory -> (architecture, checkpoint dir or None for random init)."""
    p = Path(model)
    if p.is_dir() and (p / "config.json").exists():
        with open(p / "config.json") as f:
            return _from_hf_config(json.load(f), model), p
    hf_home = os.environ.get("HF_HOME")
    if hf_home:
        snap = Path(hf_home) / "hub" / ("models--" + model.replace("/", "--")) / "snapshots"
        if snap.is_dir():
            for d in sorted(snap.iterdir()):
                if (d / "config.json").exists():
                    with open(d / "config.json") as f:
                        return _from_hf_config(json.load(f), model), d
    key = model.lower()
    key = _ALIASES.get(key, key)
    base = key.split("/")[-1]
    for cand in (key, base):
        if cand in PRESETS:
            cfg = PRESETS[cand]
            return ModelConfig(**{**cfg.__dict__, "name": model}), None
    for preset in PRESETS:
        if preset in base:
            cfg = PRESETS[preset]
            return ModelConfig(**{**cfg.__dict__, "name": model}), None
    raise ValueError(f"unknown model {model!r}: not a checkpoint directory and not a known architecture")


_DTYPES = {"auto": torch.bfloat16, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float16": torch.float16, "half": torch.float16, "float32": torch.float32,
           "float": torch.float32}


@dataclass
class KVTransferConfig:
    """--kv-transfer-config JSON (kv_connector / kv_role / kv_connector_extra_config)."""
    kv_connector: str = ""
    kv_role: str = "kv_both"  # kv_both | kv_producer | kv_consumer
    extra: dict = field(default_factory=dict)

    @classmethod
    def from_json(cls, s: str | None) -> "KVTransferConfig | None":
        if not s:
            return None
        d = json.loads(s)
        return cls(d.get("kv_connector", ""), d.get("kv_role", "kv_both"),
                   d.get("kv_connector_extra_config", {}) or {})


@dataclass
class KVOffloadConfig:
    """Tiered KV settings; field names follow the LMCACHE_* env contract."""
    local_cpu: bool = False
    max_local_cpu_gb: float = 0.0
    max_local_disk_gb: float = 0.0
    local_disk_path: str = "/tmp/vpsa_kv_disk"
    remote_url: str | None = None  # lm://host:port
    remote_serde: str = "naive"  # naive | cachegen
    chunk_tokens: int = 256
    enable_controller: bool = False
    instance_id: str = ""
    controller_url: str | None = None
    worker_port: int = 0
    distributed_url: str | None = None
    enable_pd: bool = False  # LMCACHE_ENABLE_NIXL
    pd_role: str = ""  # sender | receiver
    pd_peer_host: str = ""
    pd_peer_port: int = 55555
    pd_buffer_bytes: int = 1 << 30
    pd_buffer_device: str = "hip"

    @classmethod
    def from_env(cls, env: dict[str, str] | None = None) -> "KVOffloadConfig":
        e = os.environ if env is None else env

        def flag(k: str) -> bool:
            return str(e.get(k, "")).strip().lower() in ("1", "true", "yes", "on")

        def num(k: str, d: float = 0.0) -> float:
            try:
                return float(e.get(k, d))
            except (TypeError, ValueError):
                return d

        return cls(
            local_cpu=flag("LMCACHE_LOCAL_CPU"),
            max_local_cpu_gb=num("LMCACHE_MAX_LOCAL_CPU_SIZE"),
            max_local_disk_gb=num("LMCACHE_MAX_LOCAL_DISK_SIZE"),
            local_disk_path=e.get("LMCACHE_LOCAL_DISK", "/tmp/vpsa_kv_disk").replace("file://", ""),
            remote_url=e.get("LMCACHE_REMOTE_URL") or None,
            remote_serde=(e.get("LMCACHE_REMOTE_SERDE") or "naive").lower(),
            chunk_tokens=int(num("LMCACHE_CHUNK_SIZE", 256)),
            enable_controller=flag("LMCACHE_ENABLE_CONTROLLER"),
            instance_id=e.get("LMCACHE_LMCACHE_INSTANCE_ID", ""),
            controller_url=e.get("LMCACHE_CONTROLLER_URL") or None,
            worker_port=int(num("LMCACHE_LMCACHE_WORKER_PORT", 0)),
            distributed_url=e.get("LMCACHE_DISTRIBUTED_URL") or None,
            enable_pd=flag("LMCACHE_ENABLE_NIXL"),
            pd_role=e.get("LMCACHE_NIXL_ROLE", ""),
            pd_peer_host=e.get("LMCACHE_NIXL_RECEIVER_HOST", e.get("LMCACHE_NIXL_PEER_HOST", "")),
            pd_peer_port=int(num("LMCACHE_NIXL_RECEIVER_PORT", num("LMCACHE_NIXL_PEER_PORT", 55555))),
            pd_buffer_bytes=int(num("LMCACHE_NIXL_BUFFER_SIZE", 1 << 30)),
            pd_buffer_device=e.get("LMCACHE_NIXL_BUFFER_DEVICE", "hip"),
        )

    @property
    def enabled(self) -> bool:
        return bool(self.local_cpu or self.max_local_disk_gb > 0 or self.remote_url)


@dataclass
class EngineConfig:
    model: str = "tiny-llama"
    served_model_name: str | None = None
    host: str = "0.0.0.0"
    port: int = 8000
    dtype: str = "auto"
    device: str = "auto"
    max_model_len: int | None = None
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 8192
    gpu_memory_utilization: float = 0.9
    num_gpu_blocks_override: int | None = None
    enable_prefix_caching: bool = True
    enable_chunked_prefill: bool = True
    tensor_parallel_size: int = 1
    pipeline_parallel_size: int = 1
    enable_expert_parallel: bool = False  # MoE layers: whole experts per tensor-parallel rank
    # decode steps launched back to back before the host looks at the sampled tokens (greedy
    # decode-only batches of a single-rank replica with nothing waiting; 1 = every step)
    num_scheduler_steps: int = 1
    # KV pool allocated as this many pools of consecutive layers (a decode step of one layer then
    # walks a shorter address range); 0 = 4 for a large GPU pool on a replica without lower KV tiers
    # and without page transfers to or from other replicas, else 1.  Lower tiers work with any value
    # (their copies are then per piece); replicas that exchange pages always keep whole pages.
    kv_layer_groups: int = 0
    distributed_executor_backend: str | None = None
    enable_lora: bool = False
    max_loras: int = 1
    max_lora_rank: int = 16
    enable_sleep_mode: bool = False
    enable_auto_tool_choice: bool = False
    tool_call_parser: str | None = None
    chat_template: str | None = None
    kv_transfer: KVTransferConfig | None = None
    kv_offload: KVOffloadConfig = field(default_factory=KVOffloadConfig)
    swap_space: float = 0.0
    enforce_eager: bool = False
    capture_graphs_at_start: bool = True  # HIP graphs for all decode batch buckets at start-up
    # second copy of the dense MLP matrices in matrix-core tile order, streamed by decode-only steps
    # (Llama-3-8B, 40 sequences: decode step 23.0 -> 22.75 ms for 11 GiB of HBM, so off by default):
    # "off", "on", "auto" = on when it costs at most a tenth of the card's memory
    packed_decode_weights: str = "off"
    # Latency-aware prefill admission: after the first prefill of a step, more waiting requests
    # join only while the estimated prefill time of the step stays under this many ms
    # (0 = fill the token budget).  The estimate prices GEMM and attention FLOPs at the rates
    # below (what the library GEMM and the prefill attention kernel sustain on one MI355X).
    prefill_step_ms: float = 30.0
    gemm_tflops_estimate: float = 1500.0
    attn_tflops_estimate: float = 900.0
    seed: int = 0
    api_key: str | None = None
    disable_log_requests: bool = False
    trust_remote_code: bool = False
    task: str = "generate"
    load_format: str = "auto"  # auto | dummy

    def torch_dtype(self) -> torch.dtype:
        return _DTYPES[self.dtype.lower()]

    def resolve_device(self) -> torch.device:
        if self.device == "auto":
            if torch.cuda.is_available():
                return torch.device("cuda", torch.cuda.current_device())
            return torch.device("cpu")
        dev = torch.device(self.device)
        if dev.type == "cuda" and dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        return dev

    @property
    def model_name(self) -> str:
        return self.served_model_name or self.model
