"""The Luduvik decoder as a registry entry: its configuration, its blocks and where its
parameters are found in a safetensors file.

File names: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1``, the mixer under
``l<i>.mix.`` and the feed-forward under ``l<i>.mlp.``. A lightning mixer has ``q, k, v, g, o,
norm``; a parallel mixer has ``left.{q, k, v, q.norm, k.norm, o, out}`` and ``right.{q, k, v,
g, o, out}`` (``out``: the weight of the branch's norm over the model width). The feed-forward
has ``router``, ``router.b``, ``e<j>.{gate, up, down}`` and ``shared.{gate, up, down}``.
Projections that read the same rows are joined by rows into one matrix: q, k, v (and g); the
gate and up matrices of every expert, expert after expert; all experts' down matrices.
"""
from __future__ import annotations

from typing import Dict

from ..config.luduvik import LuduvikConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import ConfigError
from ..weights.loader import Piece, Source


def _one(name, shape):
    return Source(options=((Piece(name, tuple(shape)),),))


def _join(*pieces):
    return Source(options=(tuple(Piece(n, tuple(s)) for n, s in pieces),))


def _linear_heads(src, q, m, lin, d):
    nk, nv = lin.heads * lin.dim, lin.heads * lin.vdim
    src[q + "in.weight"] = _join((m + "q", (nk, d)), (m + "k", (nk, d)), (m + "v", (nv, d)), (m + "g", (nv, d)))
    src[q + "out.weight"] = _one(m + "o", (d, nv))


def luduvik_weight_sources(cfg: LuduvikConfig, file_format: str) -> Dict[str, Source]:
    if file_format != "safetensors":
        raise ValueError(f"Luduvik weights come as safetensors, not {file_format!r}")
    d, V = cfg.width, cfg.vocab
    src = {"embed.weight": _one("embed", (V, d)), "head.weight": _one("head", (V, d)),
           "final_norm.weight": _one("final.norm", (d,))}
    for i, l in enumerate(cfg.layers):
        f, p = f"l{i}.", f"blocks.{i}."
        src[p + "norm1.weight"] = _one(f + "norm1", (d,))
        m, q = f + "mix.", p + "mixer."
        if l.type == "lightning":
            _linear_heads(src, q, m, l.lightning, d)
            src[q + "norm.weight"] = _one(m + "norm", (l.lightning.heads * l.lightning.vdim,))
        else:
            a = l.left
            src[q + "left.qkv.weight"] = _join((m + "left.q", (a.heads * a.dim, d)),
                                               (m + "left.k", (a.kv_heads * a.dim, d)),
                                               (m + "left.v", (a.kv_heads * a.vdim, d)))
            src[q + "left.q_norm.weight"] = _one(m + "left.q.norm", (a.dim,))
            src[q + "left.k_norm.weight"] = _one(m + "left.k.norm", (a.dim,))
            src[q + "left.out.weight"] = _one(m + "left.o", (d, a.heads * a.vdim))
            _linear_heads(src, q + "right.", m + "right.", l.right, d)
            src[q + "norms.left"] = _one(m + "left.out", (d,))
            src[q + "norms.right"] = _one(m + "right.out", (d,))
        if l.mlp is not None:
            e, g, q = l.mlp, f + "mlp.", p + "ffn."
            src[q + "router.weight"] = _one(g + "router", (e.experts, d))
            src[q + "router.bias"] = _one(g + "router.b", (e.experts,))
            src[q + "experts.gate_up.weight"] = _join(*[(f"{g}e{j}.{n}", (e.ff, d))
                                                        for j in range(e.experts) for n in ("gate", "up")])
            src[q + "experts.down.weight"] = _join(*[(f"{g}e{j}.down", (d, e.ff)) for j in range(e.experts)])
            if e.shared_ff is not None:
                src[q + "shared.gate_up.weight"] = _join((g + "shared.gate", (e.shared_ff, d)),
                                                         (g + "shared.up", (e.shared_ff, d)))
                src[q + "shared.down.weight"] = _one(g + "shared.down", (d, e.shared_ff))
    return src


def _no_gguf(meta, rows=None):
    raise ConfigError("Luduvik models are read from a folder with config.json and model.safetensors")


LUDUVIK = Architecture(
    name="Luduvik",
    config_from_dict=LuduvikConfig.from_dict,
    config_from_gguf=_no_gguf,
    model_spec=lambda cfg: cfg.model_spec(),
    weight_sources=luduvik_weight_sources,
)

register_architecture(LUDUVIK, "luduvik")
