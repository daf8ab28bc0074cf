"""Typed configuration of the Saredra decoder, read from its own config.json.

A Saredra model is a list of pre-norm layers ``x <- x + mixer(n1(x))``, then ``x <- x + ff(n2(x))``
where the layer has a feed-forward. Two mixers: "attention" (grouped-query softmax attention with
key and value widths of their own, a rotation of pairs of neighbouring coordinates on part of
every head, capped scores, a sliding window, a softmax denominator with one added, a sigmoid gate
on the heads; a layer may read the keys and values that an earlier layer cached) and "parallel"
(two mixers side by side on the same rows, summed with fixed scales: softmax attention with
biases, a short causal convolution on q, k and v, slowed long wavelengths and a learned extra
term of the denominator per head; and a selective state-space mixer with a scalar decay per
head). The feed-forward is a dense gated unit or routes a token to the ``top`` experts with the
largest softmax scores among the experts of the best groups.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``layers[i].{type, mixer, mlp}``.
``mixer`` by type: attention: heads, kv_heads, dim, vdim, scale, softcap, mask.size, rot.{base,
dims, scaling.{factor, original, fast, slow}}, kv_from; parallel: ``left`` (the same keys and
``conv``), ``right.{heads, vdim, state, groups, conv, norm_groups}``, ``left_scale``,
``right_scale``. ``mlp``: null, ``{kind: "dense", ff}`` or ``{kind: "moe", router.{experts, top,
groups.{count, keep}}, expert.{ff}}``. Absent keys mean absent mechanisms: no ``rot``: no
rotation; no ``scaling``: plain frequencies; no ``mask``: every earlier token is seen; no
``softcap``: scores as they are; no ``conv``: no convolution; no ``groups``: all experts compete;
``kv_heads`` defaults to ``heads``, ``vdim`` to ``dim``, the branch scales to 1.
"""
from __future__ import annotations

import dataclasses
import math
from dataclasses import dataclass, field
from typing import Optional, Tuple

from .spec import (BlockSpec, BranchSumSpec, ConfigError, GLUSpec, ModelSpec, NormSpec, RoutedMLPSpec, RunSpec,
                   SinkAttentionSpec, StateSpaceSpec)
from .vametar import _get

LAYER_TYPES = ("attention", "parallel")
# fixed by the design: a rotation with slowed frequencies multiplies cos and sin by
# MAGNITUDE_SLOPE * ln(factor) + 1
MAGNITUDE_SLOPE = 0.1


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None     # factor, original, fast, slow

    @classmethod
    def from_dict(cls, d, where: str) -> Optional["Rotation"]:
        if d is None:
            return None
        if not isinstance(d, dict):
            raise ConfigError(f"config key '{where[:-1]}' must be an object")
        sc = d.get("scaling")
        scaling = None
        if sc is not None:
            w = where + "scaling."
            scaling = tuple(_get(sc, k, float, w) for k in ("factor", "original", "fast", "slow"))
        return cls(dims=_get(d, "dims", int, where), base=_get(d, "base", float, where), scaling=scaling)

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return d

    def magnitude(self) -> float:
        return 1.0 if self.scaling is None else MAGNITUDE_SLOPE * math.log(self.scaling[0]) + 1.0


@dataclass(frozen=True)
class SoftmaxHeads:
    """Heads of a softmax mixer: the "attention" mixer or the left branch of "parallel"."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    window: Optional[int] = None
    rot: Optional[Rotation] = None
    conv: int = 0                       # taps of the convolution on q, k, v (left branch)
    kv_from: Optional[int] = None       # the layer whose keys and values are read ("attention")

    @classmethod
    def from_dict(cls, m, where: str, left: bool) -> "SoftmaxHeads":
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where[:-1]}' is required")
        heads, dim = _get(m, "heads", int, where), _get(m, "dim", int, where)
        mask = m.get("mask")
        return cls(heads=heads, kv_heads=_get(m, "kv_heads", int, where, heads), dim=dim,
                   vdim=_get(m, "vdim", int, where, dim), scale=_get(m, "scale", float, where),
                   softcap=_get(m, "softcap", float, where, None),
                   window=None if mask is None else _get(mask, "size", int, where + "mask."),
                   rot=Rotation.from_dict(m.get("rot"), where + "rot."),
                   conv=_get(m, "conv", int, where, 0) if left else 0,
                   kv_from=None if left else _get(m, "kv_from", int, where, None))

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        if self.conv:
            d["conv"] = self.conv
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d

    def layout(self):
        """What a layer that lends its keys and values shares with its readers."""
        return (self.kv_heads, self.dim, self.vdim, self.rot)


@dataclass(frozen=True)
class StateSpaceHeads:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, m, where: str) -> "StateSpaceHeads":
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where[:-1]}' is required")
        return cls(heads=_get(m, "heads", int, where), vdim=_get(m, "vdim", int, where),
                   state=_get(m, "state", int, where), groups=_get(m, "groups", int, where, 1),
                   conv=_get(m, "conv", int, where, 1), norm_groups=_get(m, "norm_groups", int, where, 1))

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)


@dataclass(frozen=True)
class FeedForward:
    kind: str                           # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0
    group_count: int = 1
    group_keep: int = 1

    @classmethod
    def from_dict(cls, m, where: str) -> Optional["FeedForward"]:
        if m is None:
            return None
        kind = m.get("kind") if isinstance(m, dict) else None
        if kind == "dense":
            return cls(kind=kind, ff=_get(m, "ff", int, where))
        if kind != "moe":
            raise ConfigError(f"config key '{where}kind' must be 'dense' or 'moe', got {kind!r}")
        r, e = m.get("router"), m.get("expert")
        g = r.get("groups") if isinstance(r, dict) else None
        return cls(kind=kind, ff=_get(e, "ff", int, where + "expert."),
                   experts=_get(r, "experts", int, where + "router."), top=_get(r, "top", int, where + "router."),
                   group_count=1 if g is None else _get(g, "count", int, where + "router.groups."),
                   group_keep=1 if g is None else _get(g, "keep", int, where + "router.groups."))

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        r = {"experts": self.experts, "top": self.top}
        if self.group_count != 1:
            r["groups"] = {"count": self.group_count, "keep": self.group_keep}
        return {"kind": "moe", "router": r, "expert": {"ff": self.ff}}


@dataclass(frozen=True)
class SaredraLayer:
    type: str
    attention: Optional[SoftmaxHeads] = None        # type "attention"
    left: Optional[SoftmaxHeads] = None             # type "parallel": the softmax branch
    right: Optional[StateSpaceHeads] = None         # type "parallel": the state-space branch
    left_scale: float = 1.0
    right_scale: float = 1.0
    mlp: Optional[FeedForward] = None

    @classmethod
    def from_dict(cls, d, i: int) -> "SaredraLayer":
        where = f"layers[{i}]."
        typ = d.get("type") if isinstance(d, dict) else None
        if typ not in LAYER_TYPES:
            raise ConfigError(f"config key '{where}type' must be one of {LAYER_TYPES}, got {typ!r}")
        m = d.get("mixer")
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where}mixer' is required")
        mlp = FeedForward.from_dict(d.get("mlp"), where + "mlp.")
        if typ == "attention":
            return cls(type=typ, attention=SoftmaxHeads.from_dict(m, where + "mixer.", left=False), mlp=mlp)
        return cls(type=typ, left=SoftmaxHeads.from_dict(m.get("left"), where + "mixer.left.", left=True),
                   right=StateSpaceHeads.from_dict(m.get("right"), where + "mixer.right."),
                   left_scale=_get(m, "left_scale", float, where + "mixer.", 1.0),
                   right_scale=_get(m, "right_scale", float, where + "mixer.", 1.0), mlp=mlp)

    def to_dict(self) -> dict:
        if self.type == "attention":
            mixer = self.attention.to_dict()
        else:
            mixer = {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                     "right_scale": self.right_scale}
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class SaredraConfig:
    vocab: int
    width: int
    layers: Tuple[SaredraLayer, ...]
    eps: float
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    torch_dtype: Optional[str] = None
    tie_embeddings: Optional[bool] = False      # the output matrix is a tensor of its own
    architecture: str = "Saredra"

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        for i, l in enumerate(self.layers):
            w = f"layers[{i}]"
            a = l.attention if l.type == "attention" else l.left
            if min(a.heads, a.kv_heads, a.dim, a.vdim) < 1 or a.heads % a.kv_heads:
                raise ConfigError(f"{w}: {a.heads} heads of {a.dim} / {a.vdim} do not divide into {a.kv_heads} kv heads")
            if a.rot is not None and (a.rot.dims < 0 or a.rot.dims % 2 or a.rot.dims > a.dim):
                raise ConfigError(f"{w}: rot.dims {a.rot.dims} must be even and at most dim {a.dim}")
            if a.window is not None and a.window < 1:
                raise ConfigError(f"{w}: mask.size must be at least 1, got {a.window}")
            if a.softcap is not None and not a.softcap > 0:
                raise ConfigError(f"{w}: softcap must be positive, got {a.softcap}")
            if a.conv < 0:
                raise ConfigError(f"{w}: conv must not be negative, got {a.conv}")
            if a.kv_from is not None:
                j = a.kv_from
                if not 0 <= j < i or self.layers[j].type != "attention" or self.layers[j].attention.kv_from is not None:
                    raise ConfigError(f"{w}: kv_from {j} must name an earlier attention layer with keys and "
                                      f"values of its own")
                if self.layers[j].attention.layout() != a.layout():
                    raise ConfigError(f"{w}: kv_from {j}: head counts, widths and rotation must equal that layer's")
            if l.right is not None:
                r = l.right
                if min(r.heads, r.vdim, r.state, r.groups, r.conv, r.norm_groups) < 1 or r.heads % r.groups or \
                        (r.heads * r.vdim) % r.norm_groups:
                    raise ConfigError(f"{w}: state space of {r.heads} heads of {r.vdim}, state {r.state}, "
                                      f"{r.groups} groups, {r.norm_groups} norm parts, {r.conv} taps")
            if l.mlp is not None:
                m = l.mlp
                if m.ff < 1:
                    raise ConfigError(f"{w}: feed-forward of {m.ff}")
                if m.kind == "moe" and (not 1 <= m.top <= m.experts or m.group_count < 1 or m.experts % m.group_count
                                        or not 1 <= m.group_keep <= m.group_count
                                        or m.top > m.group_keep * (m.experts // m.group_count)):
                    raise ConfigError(f"{w}: top {m.top} of {m.experts} experts in {m.group_count} groups of which "
                                      f"{m.group_keep} stay")

    # ------------------------------------------------------------- config.json
    @classmethod
    def from_dict(cls, d: dict) -> "SaredraConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        eos = d.get("eos_token_id")
        stops = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        dt = d.get("torch_dtype", d.get("dtype"))
        return cls(vocab=_get(d, "vocab", int, ""), width=_get(d, "width", int, ""),
                   layers=tuple(SaredraLayer.from_dict(l, i) for i, l in enumerate(layers)),
                   eps=_get(d.get("norm"), "eps", float, "norm."), stop_ids=stops,
                   torch_dtype=dt[6:] if isinstance(dt, str) and dt.startswith("torch.") else dt)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.eps}, "layers": [l.to_dict() for l in self.layers]}
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        if self.stop_ids:
            d["eos_token_id"] = list(self.stop_ids)
        return d

    def default_engine_dtype(self) -> str:
        return "float32" if self.torch_dtype == "float32" else "bfloat16"

    def with_layers(self, n: int) -> "SaredraConfig":
        """The first n layers; a layer whose lender is cut off cannot occur (lenders come first)."""
        return dataclasses.replace(self, layers=self.layers[:int(n)])

    # ------------------------------------------------------------ model layout
    def cache_window(self, i: int) -> Optional[int]:
        """The window that layer i's cache is kept for: the widest among the layer and its readers
        (None as soon as one of them sees everything)."""
        users = [self.layers[i].attention] + [l.attention for l in self.layers
                                              if l.type == "attention" and l.attention.kv_from == i]
        if any(u.window is None for u in users):
            return None
        return max(u.window for u in users)

    def _softmax(self, a: SoftmaxHeads, left: bool, cache_window: Optional[int]) -> SinkAttentionSpec:
        rot = a.rot
        return SinkAttentionSpec(
            hidden=self.width, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim, value_dim=a.vdim,
            scale=a.scale, softcap=a.softcap, window=a.window, cache_window=0 if cache_window is None else cache_window,
            sink="learned" if left else "unit", rot_dims=rot.dims if rot else 0, rot_base=rot.base if rot else 10000.0,
            rot_style="interleaved", rot_ramp=rot.scaling if rot else None, rot_magnitude=rot.magnitude() if rot else 1.0,
            qkv_bias=left, conv_taps=a.conv, out_gate=not left, own_kv=a.kv_from is None)

    def model_spec(self) -> ModelSpec:
        d = self.width
        norm = NormSpec(size=d, eps=self.eps)
        blocks, schedule = [], []
        for i, l in enumerate(self.layers):
            if l.type == "attention":
                a = l.attention
                owner = i if a.kv_from is None else a.kv_from
                mixer = self._softmax(a, False, self.cache_window(owner))
                schedule.append(RunSpec(block=i, cache_of=a.kv_from))
            else:
                r = l.right
                right = StateSpaceSpec(hidden=d, num_heads=r.heads, head_dim=r.vdim, state=r.state, groups=r.groups,
                                       taps=r.conv, norm_groups=r.norm_groups, eps=self.eps)
                mixer = BranchSumSpec(hidden=d, branches=(self._softmax(l.left, True, l.left.window), right),
                                      names=("left", "right"), scales=(l.left_scale, l.right_scale))
                schedule.append(RunSpec(block=i))
            ffn = None
            if l.mlp is not None and l.mlp.kind == "dense":
                ffn = GLUSpec(hidden=d, intermediate=l.mlp.ff, activation="silu")
            elif l.mlp is not None:
                m = l.mlp
                ffn = RoutedMLPSpec(hidden=d, experts=m.experts, top=m.top, intermediate=m.ff, activation="silu",
                                    score="softmax", renormalize=False, weight_on="output", shared_intermediate=None,
                                    shared_gate=False, form="glu", groups=m.group_count, keep_groups=m.group_keep)
            blocks.append(BlockSpec(norm1=norm, mixer=mixer, norm2=norm if ffn is not None else None, ffn=ffn))
        spec = ModelSpec(vocab=self.vocab, hidden=d, blocks=tuple(blocks), schedule=tuple(schedule), final_norm=norm,
                         tie_embeddings=False, max_position=None, stop_ids=self.stop_ids)
        spec.validate()
        return spec
