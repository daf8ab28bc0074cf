"""Mixers side by side.

``BranchSum``: several mixers read the same rows and the block adds the sum of their results,
each times a fixed scale (``BranchSumSpec``).

``BranchMean``: several mixers read the same rows; each result is RMS-normed over the model
width with a weight vector of its own, and the mean of the normed results is what the block
adds to the stream (``BranchMeanSpec``). The branches keep their own cache layers: the
part's need is the list of theirs, in order.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import Param
from .base import Part, PartError, build_part, register_part


def _needs(part):
    need = part.cache_need()
    if need is None:
        return [], False
    if isinstance(need, (list, tuple)):
        return list(need), True
    return [need], False


class _Branches(Part):
    """What mixers side by side share: their names, cache layers in order, the first planner."""

    def _take(self, spec, dtype, device):
        if not 1 <= len(spec.branches) <= 4 or len(spec.names) != len(spec.branches) \
                or len(set(spec.names)) != len(spec.names):
            raise PartError(f"branches {spec.names!r}: one to four, each with a name of its own")
        if any(n == "norms" or "." in n for n in spec.names):
            raise PartError(f"branch names {spec.names!r}: no dots, and 'norms' is the part's own")
        self.spec, self.dtype = spec, dtype
        self.names = tuple(spec.names)
        self.branches = [build_part(b, dtype, device) for b in spec.branches]
        kinds = [b.kind for b in spec.branches]
        # two branches of one kind share their scratch names: the first one's result is put aside
        self._keep = [kinds.count(k) > 1 for k in kinds]

    def children(self):
        return dict(zip(self.names, self.branches))

    @property
    def graph_safe(self) -> bool:
        return all(getattr(b, "graph_safe", False) for b in self.branches)

    def cache_need(self):
        out = []
        for b in self.branches:
            out += _needs(b)[0]
        return out

    def step_planner(self):
        for b in self.branches:
            f = getattr(b, "step_planner", None)
            p = f() if f is not None else None
            if p is not None:
                return p
        return None

    def _run_branches(self, h, ctx, cache, layer, writes_cache):
        layers = list(layer) if isinstance(layer, (list, tuple)) else ([] if layer is None else [layer])
        deltas = []
        for i, b in enumerate(self.branches):
            need, several = _needs(b)
            mine = [layers.pop(0) for _ in need]
            delta, bias = b.run(h, ctx, cache, tuple(mine) if several else (mine[0] if mine else None),
                                writes_cache)
            if bias is not None or delta is None:
                raise PartError(f"branch {self.names[i]!r}: a branch returns its whole result as one delta")
            if self._keep[i] and i + 1 < len(self.branches):
                delta = ctx.ws.take(f"branch.keep.{i}", delta.shape, torch.float32).copy_(delta)
            deltas.append(delta)
        return deltas


class BranchSum(_Branches):
    def __init__(self, spec, dtype, device):
        self._take(spec, dtype, device)
        if len(spec.scales) != len(spec.branches):
            raise PartError(f"branches {spec.names!r}: a scale for each, got {len(spec.scales)}")
        self.scales = tuple(float(v) for v in spec.scales)

    def run(self, h, ctx, cache, layer, writes_cache=True):
        deltas = self._run_branches(h, ctx, cache, layer, writes_cache)
        out = ctx.ws.take("branch.sum", (h.shape[0], self.spec.hidden), torch.float32)
        kernels.weighted_sum(deltas, self.scales, out)
        return out, None


register_part("branch_sum", BranchSum)


class BranchMean(_Branches):
    def __init__(self, spec, dtype, device):
        self._take(spec, dtype, device)

    def params(self):
        return {f"norms.{n}": Param((self.spec.hidden,), "vector", init="around_one") for n in self.names}

    def run(self, h, ctx, cache, layer, writes_cache=True):
        deltas = self._run_branches(h, ctx, cache, layer, writes_cache)
        out = ctx.ws.take("branch.mean", (h.shape[0], self.spec.hidden), torch.float32)
        kernels.normed_mean(deltas, [self.w[f"norms.{n}"] for n in self.names], float(self.spec.eps), out)
        return out, None


register_part("branch_mean", BranchMean)
