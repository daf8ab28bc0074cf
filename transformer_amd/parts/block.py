"""Arrangement of parts in a block.

"prenorm": x += mixer(norm1(x)); x += ffn(norm2(x)), the reference's block
(models/llama/common/src/compute.rs:204-292). The adds are
carried as a pending (delta, bias) pair and folded into the next norm, so the
float32 residual stream is read and written once per norm.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Part, build_part, register_part, span


class PreNormBlock(Part):
    def __init__(self, spec, dtype, device):
        self.dtype = dtype
        self.norm1 = build_part(spec.norm1, dtype, device)
        self.mixer = build_part(spec.mixer, dtype, device)
        # a block without a feed-forward has the mixer's sublayer only
        self.ffn = build_part(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.norm2 = build_part(spec.norm2, dtype, device) if spec.ffn is not None else None

    def children(self):
        c = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            c.update(norm2=self.norm2, ffn=self.ffn)
        return c

    def cache_need(self):
        return self.mixer.cache_need()

    def step_planner(self):
        """What the mixer wants planned on the host for steps of single tokens, or None."""
        f = getattr(self.mixer, "step_planner", None)
        return f() if f is not None else None

    @property
    def graph_safe(self) -> bool:
        """True when a step of this block is a fixed sequence of kernel launches on
        fixed buffers (no host decisions that depend on the data)."""
        return all(getattr(p, "graph_safe", False) for p in self.children().values())

    # Single-token steps of a bfloat16 engine: a few-rows product in front of a norm adds to the
    # residual stream and prepares the norm itself, and the product behind it applies the
    # rows' factors, so the norm needs no kernel of its own. Both neighbours have to offer
    # it (``can_fold`` / ``takes_scaled``); any other part gets the norm's own kernel.
    folds_norms = True

    def _fusable(self, nt: int) -> bool:
        return self.dtype == torch.bfloat16 and 0 < nt <= kernels.SKINNY_MAX_ROWS

    @staticmethod
    def _offers(part, what: str, nt: int) -> bool:
        f = getattr(part, what, None)
        return f is not None and bool(f(nt))

    def entry_fold(self, x, ctx):
        """What the last product of the block in front needs to take over norm1, or None."""
        if not (self._fusable(x.shape[0]) and self._offers(self.mixer, "takes_scaled", x.shape[0])
                and hasattr(self.norm1, "fold")):
            return None
        return self.norm1.fold(x, ctx.ws.take("block.h", x.shape, self.dtype), ctx)

    def run(self, x, pending, ctx, cache, layer, writes_cache=True, after=None):
        """x: float32 residual stream [nt, hidden]; pending: (delta, bias) not yet added to
        x, (None, None), or the ``RowScale`` of an ``entry_fold`` that the block in front has
        served. after: the block that runs next, if any. Returns the new pending."""
        nt = x.shape[0]
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        kw = {}
        if isinstance(pending, kernels.RowScale):
            kw["scale"] = pending                  # h already holds the rows, not yet scaled
        else:
            with span(ctx, "norm"):
                self.norm1.run(x, h, pending[0], pending[1])
        if self.ffn is None:
            with span(ctx, "mixer"):
                return self.mixer.run(h, ctx, cache, layer, writes_cache, **kw)
        fusable = self._fusable(nt)
        if (fusable and hasattr(self.norm2, "fold") and self._offers(self.mixer, "can_fold", nt)
                and self._offers(self.ffn, "takes_scaled", nt)):
            kw["fold"] = self.norm2.fold(x, h, ctx)
        # with many rows a part whose last product can add itself to the stream is given it
        # (``can_add`` / ``into``); it returns no delta then, and the next norm only reads
        if "fold" not in kw and self._offers(self.mixer, "can_add", nt):
            kw["into"] = x
        with span(ctx, "mixer"):
            pending = self.mixer.run(h, ctx, cache, layer, writes_cache, **kw)
        kw2 = {}
        if "fold" in kw:
            kw2["scale"] = kw["fold"].scale()
        else:
            with span(ctx, "norm"):
                self.norm2.run(x, h, pending[0], pending[1])
        handover = None
        if fusable and after is not None and self._offers(self.ffn, "can_fold", nt):
            entry = getattr(after, "entry_fold", None)
            handover = entry(x, ctx) if entry is not None else None
        if handover is not None:
            with span(ctx, "ffn"):
                self.ffn.run(h, ctx, fold=handover, **kw2)
            return handover.scale()
        if self._offers(self.ffn, "can_add", nt):
            kw2["into"] = x
        with span(ctx, "ffn"):
            return self.ffn.run(h, ctx, **kw2)


register_part("prenorm", PreNormBlock)


class GatedPreNormBlock(Part):
    """x += mult * gate1 * mixer(shift(norm1(x))); x += mult * gate2 * ffn(norm2(x)).

    The gate of a sublayer is sigmoid(W h + b) of the sublayer's normed input h; the mixer reads
    the token-shifted rows. What a sublayer adds travels as a ``kernels.GatedDelta`` to the
    next norm (of this block or of the next, or the model's last), which does the add in
    float32 and normalises in the same pass. The shift keeps the sequence's last normed row
    between steps (a state row of its own, before the mixer's needs)."""
    folds_norms = False

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.hidden = spec.hidden
        self.norm1 = build_part(spec.norm1, dtype, device)
        self.mixer = build_part(spec.mixer, dtype, device)
        self.norm2 = build_part(spec.norm2, dtype, device) if spec.ffn is not None else None
        self.ffn = build_part(spec.ffn, dtype, device) if spec.ffn is not None else None

    def children(self):
        c = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            c.update(norm2=self.norm2, ffn=self.ffn)
        return c

    def params(self):
        from ..weights.loader import Param
        d, p = self.hidden, {}
        if self.spec.token_shift:
            p["shift"] = Param((d,), "vector")
        if self.spec.gated:
            p["gate1.weight"], p["gate1.bias"] = Param((d, d), "matrix"), Param((d,), "vector")
            if self.ffn is not None:
                p["gate2.weight"], p["gate2.bias"] = Param((d, d), "matrix"), Param((d,), "vector")
        return p

    def _mixer_needs(self):
        need = self.mixer.cache_need()
        if need is None:
            return []
        return list(need) if isinstance(need, (list, tuple)) else [need]

    def cache_need(self):
        from ..cache.storage import StateNeed
        own = [StateNeed((self.hidden,), torch.float32)] if self.spec.token_shift else []
        return own + self._mixer_needs()

    def step_planner(self):
        f = getattr(self.mixer, "step_planner", None)
        return f() if f is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.children().values())

    def _gate(self, h, which, ctx):
        if not self.spec.gated:
            return None, None
        from .linear import linear
        g = linear(h, self.w[which + ".weight"],
                   ctx.ws.take("block." + which, (h.shape[0], self.hidden), torch.float32))
        return g, self.w[which + ".bias"]

    def run(self, x, pending, ctx, cache, layer, writes_cache=True, after=None):
        s = self.spec
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        layers = list(layer) if isinstance(layer, (list, tuple)) else ([] if layer is None else [layer])
        hs = h
        shift_state = cache.layer_state(layers.pop(0)) if s.token_shift else None
        # a step of single tokens: the shift rides on the norm's kernel (the row before a
        # sequence's only token is its state row)
        on_norm = s.token_shift and ctx.all_single and kernels.norm_shift_fuses(self.hidden) \
            and isinstance(pending, tuple) and getattr(self.norm1, "takes_shift", False)
        with span(ctx, "norm"):
            if on_norm:
                hs = ctx.ws.take("block.hs", x.shape, self.dtype)
                self.norm1.run(x, h, pending[0], pending[1],
                               shift=(self.w["shift"], shift_state, ctx.slots, hs))
            else:
                self.norm1.run(x, h, pending[0], pending[1])
        with span(ctx, "gate"):
            gate, gbias = self._gate(h, "gate1", ctx)
            if s.token_shift and not on_norm:
                hs = kernels.token_shift(h, ctx.ws.take("block.hs", x.shape, self.dtype), self.w["shift"],
                                         shift_state, ctx.cu_q, ctx.slots)
        need = self.mixer.cache_need()
        mixer_layer = None if need is None else tuple(layers) if isinstance(need, (list, tuple)) \
            else layers[0]
        with span(ctx, "mixer"):
            delta, bias = self.mixer.run(hs, ctx, cache, mixer_layer, writes_cache)
        pending = (kernels.GatedDelta(delta, bias, gate, gbias, s.mult), None)
        if self.ffn is None:
            return pending
        with span(ctx, "norm"):
            self.norm2.run(x, h, pending[0], pending[1])
        with span(ctx, "gate"):
            gate, gbias = self._gate(h, "gate2", ctx)
        with span(ctx, "ffn"):
            delta, bias = self.ffn.run(h, ctx)
        return (kernels.GatedDelta(delta, bias, gate, gbias, s.mult), None)


register_part("gated_prenorm", GatedPreNormBlock)


class ParallelBlock(Part):
    """h = norm1(x); x += mixer(h) + ffn(h): one norm, and both sublayers read its rows
    (``ParallelBlockSpec``). The sum travels to the next norm as one pending delta: a
    feed-forward that offers ``adds_extra`` takes the mixer's delta into its own last kernel;
    for any other the two are laid side by side as planes, which the norm adds in order."""
    folds_norms = False

    def __init__(self, spec, dtype, device):
        self.dtype = dtype
        self.norm1 = build_part(spec.norm1, dtype, device)
        self.mixer = build_part(spec.mixer, dtype, device)
        self.ffn = build_part(spec.ffn, dtype, device) if spec.ffn is not None else None

    def children(self):
        c = {"norm1": self.norm1, "mixer": self.mixer}
        if self.ffn is not None:
            c["ffn"] = self.ffn
        return c

    def cache_need(self):
        return self.mixer.cache_need()

    def step_planner(self):
        f = getattr(self.mixer, "step_planner", None)
        return f() if f is not None else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in self.children().values())

    def run(self, x, pending, ctx, cache, layer, writes_cache=True, after=None):
        if not isinstance(pending, tuple):
            raise ValueError("a parallel block takes a pending (delta, bias) pair from the block in front")
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        with span(ctx, "norm"):
            self.norm1.run(x, h, pending[0], pending[1])
        with span(ctx, "mixer"):
            delta, bias = self.mixer.run(h, ctx, cache, layer, writes_cache)
        if self.ffn is None:
            return delta, bias
        with span(ctx, "ffn"):
            if getattr(self.ffn, "adds_extra", False):
                fd, fb = self.ffn.run(h, ctx, extra=delta)
            else:
                fd, fb = self.ffn.run(h, ctx)
                planes = [t for d in (delta, fd) for t in (d if d.dim() == 3 else d.unsqueeze(0))]
                both = ctx.ws.take("block.sum", (len(planes), *x.shape), torch.float32)
                for i, t in enumerate(planes):
                    both[i].copy_(t)
                fd = both
        if bias is not None and fb is not None:
            raise ValueError("a parallel block carries one pending bias row, and both sublayers left one")
        return fd, bias if bias is not None else fb


register_part("parallel_prenorm", ParallelBlock)
