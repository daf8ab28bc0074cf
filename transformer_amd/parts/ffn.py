"""The dense SwiGLU feed-forward.

gate_up = h @ Wgu^T with the gate rows first and the up rows second
(models/llama/common/src/lib.rs:154-157, split at
compute.rs:286); act = silu(gate) * up (:286-288); the down projection is
added to the residual (:290-292).
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import Param
from .base import Part, PartError, register_part
from .linear import adds_in_place, linear, linear_delta


class SwiGLU(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype

    def params(self):
        s = self.spec
        p = {"gate_up.weight": Param((2 * s.intermediate, s.hidden), "matrix"),
             "down.weight": Param((s.hidden, s.intermediate), "matrix")}
        if s.bias:
            p["gate_up.bias"] = Param((2 * s.intermediate,), "vector")
            p["down.bias"] = Param((s.hidden,), "vector")
        return p

    def takes_scaled(self, nt: int) -> bool:
        return kernels.skinny_takes(nt, self.w["gate_up.weight"])

    def can_fold(self, nt: int) -> bool:
        return kernels.skinny_folds(nt, self.w["down.weight"])

    def can_add(self, nt: int) -> bool:
        return adds_in_place(nt, self.w["down.weight"])

    def run(self, h, ctx, scale=None, fold=None, into=None):
        """h: [nt, hidden] engine dtype -> (delta float32 [nt, hidden], bias row or None);
        None with ``fold``, which has then taken the result; (None, bias) with ``into``, the
        residual stream that the down projection has then added itself to. ``scale``: the rows
        of h still lack their norm's factor."""
        s, nt = self.spec, h.shape[0]
        act = ctx.ws.take("swiglu.act", (nt, s.intermediate), self.dtype)
        if scale is not None or kernels.skinny_wins(h, self.w["gate_up.weight"]):
            # few rows: the product applies the activation itself and [nt, 2*di] is never stored
            kernels.gemm_skinny(h, self.w["gate_up.weight"], act, swiglu=True,
                                bias=self.w.get("gate_up.bias"), scale=scale)
        elif h.dtype == torch.bfloat16 and kernels.mid_takes(nt, self.w["gate_up.weight"]):
            # up to 64 rows the product of our own applies the activation itself: 44 to 54 us on
            # the 8B shape where the vendor library's product and the activation's kernel take 55
            kernels.gemm_mid(h, self.w["gate_up.weight"], act, swiglu=True, bias=self.w.get("gate_up.bias"))
        else:
            gu = linear(h, self.w["gate_up.weight"],
                        ctx.ws.take("swiglu.gate_up", (nt, 2 * s.intermediate), self.dtype))
            kernels.swiglu(gu, act, self.w.get("gate_up.bias"))
        if fold is not None:
            kernels.gemm_skinny(act, self.w["down.weight"], None, bias=self.w.get("down.bias"), fold=fold)
            return None
        return (linear_delta(act, self.w["down.weight"], ctx.ws, "swiglu.delta", into=into),
                self.w.get("down.bias"))


class GLU(SwiGLU):
    """The same feed-forward with the activation as a parameter of the spec ("silu",
    "gelu_tanh"). Silu takes every path of ``SwiGLU`` (the products that apply it themselves
    included); another activation runs the product and then the activation's kernel."""

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.activation not in ("silu", "gelu_tanh"):
            raise PartError(f"unknown feed-forward activation {spec.activation!r}")
        self.activation = spec.activation

    def takes_scaled(self, nt: int) -> bool:
        return self.activation == "silu" and super().takes_scaled(nt)

    def run(self, h, ctx, scale=None, fold=None, into=None):
        if self.activation == "silu":
            return super().run(h, ctx, scale=scale, fold=fold, into=into)
        s, nt = self.spec, h.shape[0]
        gu = linear(h, self.w["gate_up.weight"],
                    ctx.ws.take("swiglu.gate_up", (nt, 2 * s.intermediate), self.dtype))
        act = kernels.glu(gu, ctx.ws.take("swiglu.act", (nt, s.intermediate), self.dtype),
                          self.activation, self.w.get("gate_up.bias"))
        if fold is not None:
            kernels.gemm_skinny(act, self.w["down.weight"], None, bias=self.w.get("down.bias"), fold=fold)
            return None
        return (linear_delta(act, self.w["down.weight"], ctx.ws, "swiglu.delta", into=into),
                self.w.get("down.bias"))


class MLP(Part):
    """down(act(up(h))), no gate branch (``MLPSpec``)."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        if spec.activation not in kernels._ACTIVATIONS:
            raise PartError(f"unknown feed-forward activation {spec.activation!r}")
        self.spec, self.dtype = spec, dtype

    def params(self):
        s = self.spec
        return {"up.weight": Param((s.intermediate, s.hidden), "matrix"),
                "down.weight": Param((s.hidden, s.intermediate), "matrix")}

    def run(self, h, ctx):
        s, nt = self.spec, h.shape[0]
        u = linear(h, self.w["up.weight"], ctx.ws.take("mlp.up", (nt, s.intermediate), self.dtype))
        kernels.activation(u, u, s.activation)
        return linear_delta(u, self.w["down.weight"], ctx.ws, "mlp.delta"), None


class RoutedMLP(Part):
    """Every token goes through the ``top`` experts with the largest router scores and,
    optionally, a shared expert (``RoutedMLPSpec``).

    One product gives the router's float32 logits (and the shared expert's gate); the chosen
    (token, expert) pairs are ordered by expert on the GPU into a row list whose size depends
    on the number of tokens only, so a step is the same sequence of launches whatever the
    routing; the experts' products walk that list tile by tile, each tile with its expert's
    matrix; the rows go back to their tokens in float32."""
    graph_safe = True
    adds_extra = True       # ``run(..., extra=)``: the last kernel also adds another sublayer's delta

    def __init__(self, spec, dtype, device):
        s = spec
        if not 1 <= s.top <= s.experts or s.intermediate < 1:
            raise PartError(f"routed feed-forward: top {s.top} of {s.experts} experts of {s.intermediate}")
        form = getattr(s, "form", "mlp")
        if form not in ("mlp", "limited_glu", "glu"):
            raise PartError(f"routed feed-forward: unknown form {form!r}")
        self.limited = form == "limited_glu"
        self.glu = form == "glu"                  # act(gate) * up, no limits
        self.two = self.limited or self.glu       # an expert's first matrix is [gate rows | up rows]
        self.groups, self.keep_groups = int(getattr(s, "groups", 1)), int(getattr(s, "keep_groups", 1))
        if self.groups < 1 or s.experts % self.groups or not 1 <= self.keep_groups <= self.groups or \
                s.top > self.keep_groups * (s.experts // self.groups):
            raise PartError(f"routed feed-forward: {s.experts} experts in {self.groups} groups of which "
                            f"{self.keep_groups} stay do not hold {s.top} choices")
        if self.glu:
            if s.activation not in kernels._GLU_ACTS:
                raise PartError(f"unknown expert activation {s.activation!r}")
            if s.shared_intermediate is not None:
                raise PartError("routed feed-forward: the glu form has no shared expert")
        elif self.limited:
            if not s.limit > 0 or (s.shared_intermediate is not None and not s.shared_limit > 0):
                raise PartError(f"routed feed-forward: limits must be positive, got {s.limit} / {s.shared_limit}")
        elif s.activation not in kernels._MOE_ACTS or s.activation not in kernels._ACTIVATIONS:
            raise PartError(f"unknown expert activation {s.activation!r}")
        if s.score not in ("sigmoid", "softmax") or s.weight_on not in ("input", "output"):
            raise PartError(f"routed feed-forward: score {s.score!r}, weight on {s.weight_on!r}")
        self.spec, self.dtype = s, dtype
        self.gated_shared = s.shared_intermediate is not None and s.shared_gate

    def params(self):
        s = self.spec
        # limited_glu, glu: an expert's first matrix is [gate rows | up rows]
        first, k = ("gate_up", 2) if self.two else ("up", 1)
        p = {"router.weight": Param((s.experts + int(self.gated_shared), s.hidden), "matrix"),
             f"experts.{first}.weight": Param((s.experts * k * s.intermediate, s.hidden), "matrix"),
             "experts.down.weight": Param((s.experts * s.hidden, s.intermediate), "matrix")}
        if getattr(s, "router_bias", False):
            p["router.bias"] = Param((s.experts,), "vector")
        if s.shared_intermediate is not None:
            p[f"shared.{first}.weight"] = Param((k * s.shared_intermediate, s.hidden), "matrix")
            p["shared.down.weight"] = Param((s.hidden, s.shared_intermediate), "matrix")
        return p

    def _first(self, a, w, tile_expert, ws, name, n, act_limit):
        """The first product of the experts (tile_expert given) or of the shared expert with
        its activation: rows [.., n] in the engine's type."""
        s, rows = self.spec, a.shape[0]
        k = 2 if self.two else 1
        pre = ws.take(name + ".pre", (rows, k * n), self.dtype)
        if tile_expert is not None:
            kernels.moe_gemm(a, w, tile_expert, pre, None if self.two else s.activation)
        else:
            linear(a, w, pre)
        if self.glu:
            return kernels.glu(pre, ws.take(name, (rows, n), self.dtype), s.activation)
        if not self.limited:
            if tile_expert is None:
                kernels.activation(pre, pre, s.activation)
            return pre
        return kernels.glu_limit(pre, ws.take(name, (rows, n), self.dtype), float(act_limit),
                                 float(s.gate_slope), float(s.up_shift))

    def run(self, h, ctx, extra=None):
        s, nt, d = self.spec, h.shape[0], self.spec.hidden
        E, top, ff = s.experts, s.top, s.intermediate
        ws = ctx.ws
        logits = linear(h, self.w["router.weight"], ws.take("moe.logits", (nt, E + int(self.gated_shared)), torch.float32))
        chosen = ws.take("moe.chosen", (nt, top), torch.int32)
        weight = ws.take("moe.weight", (nt, top), torch.float32)
        kernels.moe_route(logits, E, top, chosen, weight, s.score, s.renormalize, bias=self.w.get("router.bias"),
                          groups=self.groups, keep_groups=self.keep_groups)
        if getattr(ctx, "dump", None) is not None:
            ctx.dump("experts", chosen)
        rows = kernels.moe_max_rows(nt * top, E)
        row_pair = ws.take("moe.row_pair", (rows,), torch.int32)
        tile_expert = ws.take("moe.tile_expert", (rows // 16,), torch.int32)
        pair_row = ws.take("moe.pair_row", (nt * top,), torch.int32)
        kernels.moe_plan(chosen, E, row_pair, tile_expert, pair_row)
        on_input = s.weight_on == "input"
        a = kernels.moe_gather(h, top, row_pair, weight if on_input else None, ws.take("moe.a", (rows, d), self.dtype))
        first, k = ("gate_up", 2) if self.two else ("up", 1)
        up = self.w[f"experts.{first}.weight"].view(E, k * ff, d)
        down = self.w["experts.down.weight"].view(E, d, ff)
        if up.dtype != self.dtype:
            raise PartError(f"the experts' matrices are {up.dtype}, the engine computes in {self.dtype}")
        mid = self._first(a, up, tile_expert, ws, "moe.mid", ff, getattr(s, "limit", 0.0))
        out = kernels.moe_gemm(mid, down, tile_expert, ws.take("moe.out", (rows, d), torch.float32))
        shared = None
        if s.shared_intermediate is not None:
            u = self._first(h, self.w[f"shared.{first}.weight"], None, ws, "moe.shared_up", s.shared_intermediate,
                            getattr(s, "shared_limit", 0.0))
            shared = linear_delta(u, self.w["shared.down.weight"], ws, "moe.shared")
        delta = kernels.moe_combine(out, top, pair_row, None if on_input else weight, shared,
                                    logits[:, E:] if self.gated_shared else None,
                                    ws.take("moe.delta", (nt, d), torch.float32), extra=extra)
        return delta, None


register_part("swiglu", SwiGLU)
register_part("mlp", MLP)
register_part("routed_mlp", RoutedMLP)
register_part("glu", GLU)
