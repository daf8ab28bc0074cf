"""Position encodings of the attention mixer.

Interface: ``encode_and_store(qkv, ctx, nq, nkv, dest, kcache, vcache, bias)``
transforms the q and k heads of the packed qkv rows for the absolute positions
of the step (``ctx.positions``) and stores the step's k and v into the cache layer. Both happen in
one kernel because each touches every k element once.

Rotary: pair (u, v) of a head becomes (u cos a - v sin a, u sin a + v cos a) with
a = position * theta^(-2j/head_dim); the angle, sine and cosine are float32.
The reference rotates q and k in place before the cache write and hands theta to
the operator (models/llama/common/src/compute.rs:232-233,
:457-488); positions of a request are pos .. pos+seq_len (:188-198).
"""
from __future__ import annotations

import numpy as np
import torch

from .. import kernels
from .base import Part, PartError, register_part


def scaled_frequencies(dims: int, base: float, scaling=None) -> np.ndarray:
    """f_j = base^(-2j/dims), j < dims/2, float64. scaling (factor, low, high, original) slows
    the long wavelengths l = 2 pi / f: f / factor where l > original/low, f where l <
    original/high, and between the two (1 - s) f / factor + s f with s = (original/l - low) /
    (high - low)."""
    j = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * j / dims)
    if scaling is None:
        return f
    factor, low, high, original = (float(v) for v in scaling)
    if not (factor > 0 and original > 0 and high > low >= 0):
        raise PartError(f"rotary scaling: factor {factor}, low {low}, high {high}, original {original}")
    wavelength = 2.0 * np.pi / f
    share = np.clip((original / wavelength - low) / (high - low), 0.0, 1.0)
    blended = (1.0 - share) * f / factor + share * f
    return np.where(wavelength < original / high, f, np.where(wavelength > original / low, f / factor, blended))


RAMP_FLOOR = 0.001      # least width of a ramp between kept and slowed frequencies


def ramp_frequencies(dims: int, base: float, ramp) -> np.ndarray:
    """f_j = base^(-2j/dims), j < dims/2, float64, slowed along a ramp over the pair index: with
    ramp = (factor, original, fast, slow) and n(t) = dims * ln(original / (2 pi t)) / (2 ln base), lo =
    max(floor(n(fast)), 0), hi = min(ceil(n(slow)), dims - 1), r_j = clamp((j - lo) / max(hi - lo,
    RAMP_FLOOR), 0, 1): f_j <- f_j / factor * r_j + f_j * (1 - r_j)."""
    j = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * j / dims)
    factor, original, fast, slow = (float(v) for v in ramp)
    if not (factor > 0 and original > 0 and fast > 0 and slow > 0 and base > 1):
        raise PartError(f"rotary ramp: factor {factor}, original {original}, fast {fast}, slow {slow}, base {base}")

    def index(turns):
        return dims * np.log(original / (2.0 * np.pi * turns)) / (2.0 * np.log(float(base)))

    lo = max(float(np.floor(index(fast))), 0.0)
    hi = min(float(np.ceil(index(slow))), dims - 1.0)
    r = np.clip((j - lo) / max(hi - lo, RAMP_FLOOR), 0.0, 1.0)
    return f / factor * r + f * (1.0 - r)


class Rotary(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        if spec.head_dim % 2:
            raise PartError(f"rotary head size {spec.head_dim} must be even")
        if spec.style not in ("half", "interleaved"):
            raise PartError(f"unknown rotary pairing {spec.style!r}")
        self.head_dim = spec.head_dim
        self.interleaved = spec.style == "interleaved"
        scaling, ramp = getattr(spec, "scaling", None), getattr(spec, "ramp", None)
        if scaling is not None and ramp is not None:
            raise PartError("a rotation takes one way of slowing its frequencies, not both")
        if ramp is not None:
            inv = ramp_frequencies(spec.head_dim, float(spec.theta), ramp)
        else:
            inv = scaled_frequencies(spec.head_dim, float(spec.theta), scaling)
        self.inv_freq = torch.tensor(inv.astype(np.float32), device=device)
        self.magnitude = float(getattr(spec, "magnitude", 1.0))
        self.key = ("rope", spec.head_dim, float(spec.theta), None if scaling is None else tuple(scaling),
                    None if ramp is None else tuple(ramp), self.magnitude)

    def angles(self, ctx):
        """(cos, sin) of every token of the step, computed once per step and shared
        by all layers that rotate with the same frequencies."""
        table = ctx.shared.get(self.key)
        if table is None:
            out = ctx.ws.take("rope.angles." + ".".join(str(k) for k in self.key[1:]),
                              (ctx.nt, self.head_dim // 2, 2), torch.float32)
            table = kernels.rope_table(ctx.positions, self.inv_freq, out, self.magnitude)
            ctx.shared[self.key] = table
        return table

    def encode_and_store(self, qkv, ctx, nq, nkv, dest=None, kcache=None, vcache=None, bias=None):
        return kernels.rope_kv_write(qkv, nq, nkv, self.head_dim, self.angles(ctx),
                                     self.interleaved, dest, kcache, vcache, bias)

    def rotation_of(self, ctx):
        """(angle table, interleaved) for a kernel that rotates q and k itself. A position
        part without this method is always run through ``encode_and_store``."""
        return self.angles(ctx), self.interleaved


class NoPosition(Part):
    """Leaves q and k as they are; only the cache write happens."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.head_dim = spec.head_dim

    def encode_and_store(self, qkv, ctx, nq, nkv, dest=None, kcache=None, vcache=None, bias=None):
        return kernels.rope_kv_write(qkv, nq, nkv, self.head_dim, None, False, dest, kcache,
                                     vcache, bias)

    def rotation_of(self, ctx):
        return None, False


register_part("rope", Rotary)
register_part("none", NoPosition)
