"""Typed configuration of the Luduvik decoder, read from its own config.json.

A Luduvik model is a list of layers ``x <- x + mixer(n(x)) + ff(n(x))``: ONE norm in front of
both sublayers. Two mixers: "lightning" (linear attention with a fixed decay per head behind
silu maps, all heads normed together, a sigmoid gate) and "parallel" (softmax attention with
grouped heads, q and k normed per head and rotated on part of every head, beside a retention
branch: rotated q and k, fixed decays, every head's readout divided by its root mean square, a
silu gate; each branch's result is normed over the model width and the two are averaged). The
feed-forward, where a layer has one, routes a token to the ``top`` experts with the largest
router logits (softmax over the chosen logits) and adds a shared expert; an expert is a gated
unit whose gate and up branches are limited.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``layers[i].{type, mixer, mlp}``.
``mixer`` by type: lightning: heads, dim, vdim, decay (a number per head); parallel:
``left.{heads, kv_heads, dim, vdim, scale, rot.{base, dims, scaling.{factor, low, high,
original}}}`` and ``right.{heads, dim, vdim, decay, rot.{base, dims}}``. ``mlp``: null or
``{kind: "moe", router.{experts, top}, expert.{ff, limit}, shared.{ff, limit}}``. Absent keys
mean absent mechanisms: no ``rot``: no rotation; no ``scaling``: plain frequencies; no
``shared``: no shared expert; ``kv_heads`` defaults to ``heads`` and ``vdim`` to ``dim``.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional, Tuple

from .spec import (BranchMeanSpec, ConfigError, DecayLinearAttentionSpec, ModelSpec, NormSpec,
                   NormedAttentionSpec, ParallelBlockSpec, RoutedMLPSpec, RunSpec)
from .vametar import _get

LAYER_TYPES = ("lightning", "parallel")
# fixed by the design: an expert is g * sigmoid(GATE_SLOPE * g) * (u + UP_SHIFT)
GATE_SLOPE = 1.702
UP_SHIFT = 1.0


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None     # factor, low, high, original

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
            scaling = tuple(_get(sc, k, float, w) for k in ("factor", "low", "high", "original"))
        return cls(dims=_get(d, "dims", int, where), base=_get(d, "base", float, where), scaling=scaling)

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return d


def _decays(m, where: str, heads: int) -> Tuple[float, ...]:
    v = m.get("decay") if isinstance(m, dict) else None
    if not isinstance(v, (list, tuple)) or len(v) != heads or \
            any(isinstance(a, bool) or not isinstance(a, (int, float)) for a in v):
        raise ConfigError(f"config key '{where}decay' must list one number per head ({heads})")
    return tuple(float(a) for a in v)


@dataclass(frozen=True)
class LinearHeads:
    """Heads of a linear-attention mixer (lightning, or the retention branch)."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation] = None

    @classmethod
    def from_dict(cls, m, where: str) -> "LinearHeads":
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where[:-1]}' is required")
        heads, dim = _get(m, "heads", int, where), _get(m, "dim", int, where)
        return cls(heads=heads, dim=dim, vdim=_get(m, "vdim", int, where, dim),
                   decay=_decays(m, where, heads), rot=Rotation.from_dict(m.get("rot"), where + "rot."))

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class SoftmaxHeads:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None

    @classmethod
    def from_dict(cls, m, where: str) -> "SoftmaxHeads":
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where[:-1]}' is required")
        heads, dim = _get(m, "heads", int, where), _get(m, "dim", int, where)
        return cls(heads=heads, kv_heads=_get(m, "kv_heads", int, where, heads), dim=dim,
                   vdim=_get(m, "vdim", int, where, dim), scale=_get(m, "scale", float, where),
                   rot=Rotation.from_dict(m.get("rot"), where + "rot."))

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
             "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class RoutedExperts:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int] = None
    shared_limit: float = 0.0

    @classmethod
    def from_dict(cls, m, where: str) -> Optional["RoutedExperts"]:
        if m is None:
            return None
        kind = m.get("kind") if isinstance(m, dict) else None
        if kind != "moe":
            raise ConfigError(f"config key '{where}kind' must be 'moe', got {kind!r}")
        r, e, sh = m.get("router"), m.get("expert"), m.get("shared")
        return cls(experts=_get(r, "experts", int, where + "router."), top=_get(r, "top", int, where + "router."),
                   ff=_get(e, "ff", int, where + "expert."), limit=_get(e, "limit", float, where + "expert."),
                   shared_ff=None if sh is None else _get(sh, "ff", int, where + "shared."),
                   shared_limit=0.0 if sh is None else _get(sh, "limit", float, where + "shared."))

    def to_dict(self) -> dict:
        d = {"kind": "moe", "router": {"experts": self.experts, "top": self.top},
             "expert": {"ff": self.ff, "limit": self.limit}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


@dataclass(frozen=True)
class LuduvikLayer:
    type: str
    lightning: Optional[LinearHeads] = None       # type "lightning"
    left: Optional[SoftmaxHeads] = None           # type "parallel": the softmax branch
    right: Optional[LinearHeads] = None           # type "parallel": the retention branch
    mlp: Optional[RoutedExperts] = None

    @classmethod
    def from_dict(cls, d, i: int) -> "LuduvikLayer":
        where = f"layers[{i}]."
        typ = d.get("type") if isinstance(d, dict) else None
        if typ not in LAYER_TYPES:
            raise ConfigError(f"config key '{where}type' must be one of {LAYER_TYPES}, got {typ!r}")
        m = d.get("mixer")
        if not isinstance(m, dict):
            raise ConfigError(f"config key '{where}mixer' is required")
        mlp = RoutedExperts.from_dict(d.get("mlp"), where + "mlp.")
        if typ == "lightning":
            return cls(type=typ, lightning=LinearHeads.from_dict(m, where + "mixer."), mlp=mlp)
        return cls(type=typ, left=SoftmaxHeads.from_dict(m.get("left"), where + "mixer.left."),
                   right=LinearHeads.from_dict(m.get("right"), where + "mixer.right."), mlp=mlp)

    def to_dict(self) -> dict:
        mixer = self.lightning.to_dict() if self.type == "lightning" else \
            {"left": self.left.to_dict(), "right": self.right.to_dict()}
        return {"type": self.type, "mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _check_rot(rot: Optional[Rotation], dim: int, where: str) -> None:
    if rot is not None and (rot.dims < 0 or rot.dims % 2 or rot.dims > dim):
        raise ConfigError(f"{where}: rot.dims {rot.dims} must be even and at most dim {dim}")


@dataclass(frozen=True)
class LuduvikConfig:
    vocab: int
    width: int
    layers: Tuple[LuduvikLayer, ...]
    eps: float
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    torch_dtype: Optional[str] = None
    tie_embeddings: Optional[bool] = False      # the output matrix is a tensor of its own
    architecture: str = "Luduvik"

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        for i, l in enumerate(self.layers):
            w = f"layers[{i}]"
            for lin in (l.lightning, l.right):
                if lin is not None:
                    if min(lin.heads, lin.dim, lin.vdim) < 1:
                        raise ConfigError(f"{w}: {lin.heads} heads of {lin.dim} / {lin.vdim}")
                    if any(not 0.0 <= a <= 1.0 for a in lin.decay):
                        raise ConfigError(f"{w}: decays must lie in [0, 1], got {lin.decay}")
                    _check_rot(lin.rot, lin.dim, w)
            if l.left is not None:
                a = l.left
                if min(a.heads, a.kv_heads, a.dim, a.vdim) < 1 or a.heads % a.kv_heads:
                    raise ConfigError(f"{w}: {a.heads} heads do not divide into {a.kv_heads} kv heads")
                _check_rot(a.rot, a.dim, w)
            if l.mlp is not None:
                m = l.mlp
                if not 1 <= m.top <= m.experts or m.ff < 1 or not m.limit > 0:
                    raise ConfigError(f"{w}: top {m.top} of {m.experts} experts of {m.ff}, limit {m.limit}")
                if m.shared_ff is not None and (m.shared_ff < 1 or not m.shared_limit > 0):
                    raise ConfigError(f"{w}: shared expert of {m.shared_ff}, limit {m.shared_limit}")

    # ------------------------------------------------------------- config.json
    @classmethod
    def from_dict(cls, d: dict) -> "LuduvikConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config key 'layers' must be a list with at least one layer")
        eos = d.get("eos_token_id")
        stops = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        dt = d.get("torch_dtype", d.get("dtype"))
        return cls(vocab=_get(d, "vocab", int, ""), width=_get(d, "width", int, ""),
                   layers=tuple(LuduvikLayer.from_dict(l, i) for i, l in enumerate(layers)),
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

    def with_layers(self, n: int) -> "LuduvikConfig":
        return dataclasses.replace(self, layers=self.layers[:int(n)])

    # ------------------------------------------------------------ model layout
    def _linear(self, lin: LinearHeads, retention: bool) -> DecayLinearAttentionSpec:
        rot = lin.rot
        common = dict(hidden=self.width, num_heads=lin.heads, key_dim=lin.dim, value_dim=lin.vdim,
                      decays=lin.decay, eps=self.eps, rot_dims=rot.dims if rot else 0,
                      rot_base=rot.base if rot else 10000.0, rot_scaling=rot.scaling if rot else None)
        if retention:       # keys scaled by dim^-1/2 after the rotation, a unit norm per head, a silu gate
            return DecayLinearAttentionSpec(**common, input_activation=None, key_scale=float(lin.dim) ** -0.5,
                                            head_norm="per_head", norm_weight=False, gate_activation="silu")
        return DecayLinearAttentionSpec(**common, input_activation="silu", key_scale=1.0, head_norm="all_heads",
                                        norm_weight=True, gate_activation="sigmoid")

    def model_spec(self) -> ModelSpec:
        d = self.width
        norm = NormSpec(size=d, eps=self.eps)
        blocks = []
        for l in self.layers:
            if l.type == "lightning":
                mixer = self._linear(l.lightning, retention=False)
            else:
                a = l.left
                left = NormedAttentionSpec(hidden=d, num_heads=a.heads, num_kv_heads=a.kv_heads, key_dim=a.dim,
                                           value_dim=a.vdim, scale=a.scale, eps=self.eps, qk_norm=True,
                                           qk_norm_per_head=True, rot_dims=a.rot.dims if a.rot else 0,
                                           rot_base=a.rot.base if a.rot else 10000.0,
                                           rot_scaling=a.rot.scaling if a.rot else None)
                mixer = BranchMeanSpec(hidden=d, eps=self.eps, branches=(left, self._linear(l.right, True)),
                                       names=("left", "right"))
            ffn = None
            if l.mlp is not None:
                m = l.mlp
                ffn = RoutedMLPSpec(hidden=d, experts=m.experts, top=m.top, intermediate=m.ff, score="softmax",
                                    renormalize=True, weight_on="output", shared_intermediate=m.shared_ff,
                                    shared_gate=False, router_bias=True, form="limited_glu", limit=m.limit,
                                    shared_limit=m.shared_limit, gate_slope=GATE_SLOPE, up_shift=UP_SHIFT)
            blocks.append(ParallelBlockSpec(norm1=norm, mixer=mixer, ffn=ffn))
        spec = ModelSpec(vocab=self.vocab, hidden=d, blocks=tuple(blocks),
                         schedule=tuple(RunSpec(block=i) for i in range(len(blocks))), final_norm=norm,
                         tie_embeddings=False, max_position=None, stop_ids=self.stop_ids)
        spec.validate()
        return spec
