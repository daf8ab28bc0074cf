"""The Saredra decoder as a registry entry: its configuration, its blocks and where its
parameters are found in a safetensors file.

File names: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, the
mixer under ``l<i>.mix.`` and the feed-forward under ``l<i>.mlp.``. An attention mixer has ``q, k, v,
g, o`` (no ``k, v`` where it reads another layer's); a parallel mixer has ``left.{q, k, v}`` with
biases ``.b`` and convolution taps ``.conv``, ``left.sink``, ``left.o`` and ``right.{in, conv, conv.b,
dt_bias, A_log, D, norm, o}``. A dense feed-forward has ``gate, up, down``; a routed one ``router``
and ``e<j>.{gate, up, down}``. Projections that read the same rows are joined by rows into one
matrix: q, k, v (and g), their biases and their taps; gate and up; the gate and up matrices of every
expert, expert after expert; all experts' down matrices.
"""
from __future__ import annotations

from typing import Dict

from ..config.registry import Architecture, register_architecture
from ..config.saredra import SaredraConfig
from ..config.spec import ConfigError
from ..weights.loader import Piece, Source


def _one(name, shape):
    return Source(options=((Piece(name, tuple(shape)),),))


def _join(*pieces):
    return Source(options=(tuple(Piece(n, tuple(s)) for n, s in pieces),))


def _softmax_heads(src, q, m, a, d, gated):
    rows = [("q", a.heads * a.dim)]
    if a.kv_from is None:
        rows += [("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)]
    src[q + "in.weight"] = _join(*[(m + n, (r, d)) for n, r in rows], *([(m + "g", (a.heads * a.vdim, d))] if gated else []))
    src[q + "out.weight"] = _one(m + "o", (d, a.heads * a.vdim))
    return rows


def saredra_weight_sources(cfg: SaredraConfig, file_format: str) -> Dict[str, Source]:
    if file_format != "safetensors":
        raise ValueError(f"Saredra weights come as safetensors, not {file_format!r}")
    d, V = cfg.width, cfg.vocab
    src = {"embed.weight": _one("embed", (V, d)), "head.weight": _one("head", (V, d)),
           "final_norm.weight": _one("final.norm", (d,))}
    for i, l in enumerate(cfg.layers):
        f, p = f"l{i}.", f"blocks.{i}."
        src[p + "norm1.weight"] = _one(f + "norm1", (d,))
        m, q = f + "mix.", p + "mixer."
        if l.type == "attention":
            _softmax_heads(src, q, m, l.attention, d, gated=True)
        else:
            a, r = l.left, l.right
            rows = _softmax_heads(src, q + "left.", m + "left.", a, d, gated=False)
            src[q + "left.in.bias"] = _join(*[(f"{m}left.{n}.b", (n_rows,)) for n, n_rows in rows])
            if a.conv:
                src[q + "left.conv.weight"] = _join(*[(f"{m}left.{n}.conv", (n_rows, a.conv)) for n, n_rows in rows])
            src[q + "left.sink"] = _one(m + "left.sink", (a.heads,))
            inner, gn = r.heads * r.vdim, r.groups * r.state
            g = m + "right."
            src[q + "right.in.weight"] = _one(g + "in", (2 * inner + 2 * gn + r.heads, d))
            src[q + "right.conv.weight"] = _one(g + "conv", (inner + 2 * gn, r.conv))
            src[q + "right.conv.bias"] = _one(g + "conv.b", (inner + 2 * gn,))
            for n in ("dt_bias", "A_log", "D"):
                src[q + "right." + n] = _one(g + n, (r.heads,))
            src[q + "right.norm.weight"] = _one(g + "norm", (inner,))
            src[q + "right.out.weight"] = _one(g + "o", (d, inner))
        if l.mlp is not None:
            e, g, q = l.mlp, f + "mlp.", p + "ffn."
            src[p + "norm2.weight"] = _one(f + "norm2", (d,))
            if e.kind == "dense":
                src[q + "gate_up.weight"] = _join((g + "gate", (e.ff, d)), (g + "up", (e.ff, d)))
                src[q + "down.weight"] = _one(g + "down", (d, e.ff))
            else:
                src[q + "router.weight"] = _one(g + "router", (e.experts, d))
                src[q + "experts.gate_up.weight"] = _join(*[(f"{g}e{j}.{n}", (e.ff, d))
                                                            for j in range(e.experts) for n in ("gate", "up")])
                src[q + "experts.down.weight"] = _join(*[(f"{g}e{j}.down", (d, e.ff)) for j in range(e.experts)])
    return src


def _no_gguf(meta, rows=None):
    raise ConfigError("Saredra models are read from a folder with config.json and model.safetensors")


SAREDRA = Architecture(
    name="Saredra",
    config_from_dict=SaredraConfig.from_dict,
    config_from_gguf=_no_gguf,
    model_spec=lambda cfg: cfg.model_spec(),
    weight_sources=saredra_weight_sources,
)

register_architecture(SAREDRA, "saredra")
