"""The attention mixer: qkv projection, position encoding fused with the cache
write, causal grouped-query attention over the cache, output projection.

Order and shapes follow the reference's block
(models/llama/common/src/compute.rs:210-270): one merged qkv
product whose rows are all q heads, then all k heads, then all v heads
(lib.rs:132-137, split at compute.rs:227); rotation of q and k (:232-233); per
request, the step's k and v go to cache rows pos..pos+seq and the queries read
rows 0..pos+seq (:243-264); the output projection is added to the residual
(:267-270). Scale and mask are not arguments there (:511-526); here the scale
and the window are constants of the spec.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels
from ..cache.storage import KVNeed
from ..weights.loader import Param
from .base import Part, PartError, build_part, register_part
from .linear import adds_in_place, linear, linear_delta


@dataclass(frozen=True)
class KeyUnitPlanner:
    """The work plan of the single-token attention kernels, made on the host with every step's
    tables: the sequences of the step cut into units of work of about equal length
    (``kernels.plan_key_units``). Mixers with the same number of kv heads share one plan."""
    num_kv_heads: int

    def ints(self, batch: int) -> int:
        return kernels.UNIT_INTS * kernels.key_unit_count(batch, self.num_kv_heads) + 2 * batch

    def tables(self, kv_lens, block_table):
        units, seq_units = kernels.plan_key_units(
            kv_lens, kernels.key_unit_count(len(kv_lens), self.num_kv_heads), tables=block_table)
        return {"units": units, "seq_units": seq_units}


class CachedAttention(Part):
    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.position, "graph_safe", False))

    def __init__(self, spec, dtype, device):
        if spec.num_heads % spec.num_kv_heads:
            raise PartError(f"{spec.num_heads} heads do not divide into {spec.num_kv_heads} kv heads")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
            raise PartError(f"attention kernels take head sizes that are multiples of 16 in "
                            f"[16, 256], not {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise PartError(f"attention window must be >= 1, got {spec.window}")
        self.spec, self.dtype = spec, dtype
        self.nq, self.nkv, self.dh = spec.num_heads, spec.num_kv_heads, spec.head_dim
        self.position = build_part(spec.position, dtype, device)

    def params(self):
        s = self.spec
        width = (self.nq + 2 * self.nkv) * self.dh
        p = {"qkv.weight": Param((width, s.hidden), "matrix"),
             "out.weight": Param((s.hidden, self.nq * self.dh), "matrix")}
        if s.qkv_bias:
            p["qkv.bias"] = Param((width,), "vector")
        if s.out_bias:
            p["out.bias"] = Param((s.hidden,), "vector")
        return p

    def cache_need(self):
        return KVNeed(self.nkv, self.dh, self.spec.window)

    def step_planner(self):
        return KeyUnitPlanner(self.nkv)

    # a block may leave the norm in front of this part to the first product (``scale``) and
    # the norm behind it to the last (``fold``) when the few-rows product takes them
    def takes_scaled(self, nt: int) -> bool:
        return kernels.skinny_takes(nt, self.w["qkv.weight"])

    def can_fold(self, nt: int) -> bool:
        return kernels.skinny_folds(nt, self.w["out.weight"])

    # with many rows the last product can add itself to the residual stream (``into``)
    def can_add(self, nt: int) -> bool:
        return adds_in_place(nt, self.w["out.weight"])

    def _out(self, o, ctx, fold, into):
        if fold is not None:
            kernels.gemm_skinny(o, self.w["out.weight"], None, bias=self.w.get("out.bias"), fold=fold)
            return None
        return (linear_delta(o, self.w["out.weight"], ctx.ws, "attention.delta", into=into),
                self.w.get("out.bias"))

    def run(self, h, ctx, cache, layer, writes_cache=True, scale=None, fold=None, into=None):
        """h: [nt, hidden] engine dtype -> (delta float32 [nt, hidden], bias row or None);
        None with ``fold``, which has then taken the result; (None, bias) with ``into``, the
        residual stream that the output projection has then added itself to."""
        nt = h.shape[0]
        width = (self.nq + 2 * self.nkv) * self.dh
        qkv = linear(h, self.w["qkv.weight"], ctx.ws.take("attention.qkv", (nt, width), self.dtype),
                     scale=scale)
        kc, vc, group = cache.layer_kv(layer)
        meta = ctx.kv[group]
        o = ctx.ws.take("attention.o", (nt, self.nq * self.dh), self.dtype)
        fused = getattr(self.position, "rotation_of", None)
        if (ctx.all_single and fused is not None and qkv.dtype == torch.bfloat16
                and kernels.keys_kernel_fits(self.nq, self.nkv, self.dh)):
            # one token per sequence: rotation, cache write and attention in one kernel
            angles, interleaved = fused(ctx)
            plan = meta.plans.get(self.step_planner(), {})    # absent: the kernel's wrapper plans
            kernels.attention_keys(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0,
                                   ctx.max_kv_len, self.nq, self.nkv, self.dh,
                                   float(self.spec.scale), self.spec.window, angles=angles,
                                   interleaved=interleaved, bias=self.w.get("qkv.bias"),
                                   dest=meta.dest if writes_cache else None,
                                   units=plan.get("units"), seq_units=plan.get("seq_units"))
            return self._out(o, ctx, fold, into)
        if writes_cache:
            self.position.encode_and_store(qkv, ctx, self.nq, self.nkv, meta.dest, kc, vc,
                                           self.w.get("qkv.bias"))
        else:   # this run reads keys and values that an earlier run stored
            self.position.encode_and_store(qkv, ctx, self.nq, self.nkv,
                                           bias=self.w.get("qkv.bias"))
        kernels.attention(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen,
                          ctx.max_kv_len, self.nq, self.nkv, self.dh, float(self.spec.scale),
                          self.spec.window)
        return self._out(o, ctx, fold, into)


register_part("attention", CachedAttention)


class NormedAttention(Part):
    """Attention whose q and k are RMS-normed over the whole projection, rotated on part of
    every head, and whose values have a width of their own and may be mixed with the values
    an earlier layer formed for the same token (``NormedAttentionSpec``).

    One merged product gives [q | k | v]; ``kernels.qk_prepare`` does norm, rotation, value
    mixing and the cache write in one pass; attention over the paged cache follows, then the
    output projection. The values a "source" layer formed stay in ``ctx.shared`` for the
    step's later layers."""
    graph_safe = True
    _SHARED = "attention_normed.source_values"

    def __init__(self, spec, dtype, device):
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise PartError(f"{s.num_heads} heads do not divide into {s.num_kv_heads} kv heads")
        if not (1 <= s.key_dim <= 256 and 1 <= s.value_dim <= 256):
            raise PartError(f"attention takes key and value widths in [1, 256], not {s.key_dim} / {s.value_dim}")
        if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.key_dim:
            raise PartError(f"{s.rot_dims} rotated coordinates do not fit heads of {s.key_dim}")
        if s.value_mix not in (None, "source", "mix"):
            raise PartError(f"unknown value_mix {s.value_mix!r}")
        if s.window is not None and s.window < 1:
            raise PartError(f"attention window must be >= 1, got {s.window}")
        self.spec, self.dtype = s, dtype
        self.nq, self.nkv, self.dk, self.dv = s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim
        self.width = (self.nq + self.nkv) * self.dk + self.nkv * self.dv
        self.per_head = bool(getattr(s, "qk_norm_per_head", False))
        self.rotary = None
        if s.rot_dims:
            from ..config.spec import PositionSpec
            self.rotary = build_part(PositionSpec(head_dim=s.rot_dims, theta=s.rot_base, style="half",
                                                  scaling=getattr(s, "rot_scaling", None)), dtype, device)

    def params(self):
        s = self.spec
        p = {"qkv.weight": Param((self.width, s.hidden), "matrix"),
             "out.weight": Param((s.hidden, self.nq * self.dv), "matrix")}
        if s.qk_norm:
            # one weight per coordinate of the projection, or (per head) one of the head's width
            p["q_norm.weight"] = Param((self.dk if self.per_head else self.nq * self.dk,), "vector", init="around_one")
            p["k_norm.weight"] = Param((self.dk if self.per_head else self.nkv * self.dk,), "vector", init="around_one")
        if s.value_mix is not None:
            p["value_mix"] = Param((), "vector", init="zero")    # a source holds it too, unused
        return p

    # bfloat16 with a key width the matrix-core kernels take and values no wider than the keys:
    # the cache keeps value rows of the keys' width (the rest zero), so that the kernels for
    # equal widths serve prompts and single tokens, and the output projection reads the heads'
    # rows through a copy of its matrix with zero columns in the same places. Everything else
    # (float32, other widths) runs the vector-ALU kernel on values of their own width.
    def _on_matrix_cores(self) -> bool:
        return (self.dtype == torch.bfloat16 and self.dk % 32 == 0 and 32 <= self.dk <= 256
                and self.dv <= self.dk and self.width % 8 == 0)     # rows of [q | k | v] start on 16 bytes

    def cache_need(self):
        return KVNeed(self.nkv, self.dk, self.spec.window, self.dk if self._on_matrix_cores() else self.dv)

    def step_planner(self):
        if self._on_matrix_cores() and kernels.keys_kernel_fits(self.nq, self.nkv, self.dk):
            return KeyUnitPlanner(self.nkv)
        return None

    def bind(self, tensors):
        super().bind(tensors)
        self.out_wide = None
        if self._on_matrix_cores() and self.dv < self.dk and tensors["out.weight"].is_cuda:
            w = tensors["out.weight"]
            wide = torch.zeros(w.shape[0], self.nq, self.dk, dtype=w.dtype, device=w.device)
            wide[:, :, :self.dv] = w.view(w.shape[0], self.nq, self.dv)
            self.out_wide = wide.view(w.shape[0], self.nq * self.dk)

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt = self.spec, h.shape[0]
        qkv = linear(h, self.w["qkv.weight"], ctx.ws.take("attention.qkv", (nt, self.width), self.dtype))
        kc, vc, group = cache.layer_kv(layer)
        meta = ctx.kv[group]
        nv = self.nkv * self.dv
        keep = first = mix = None
        if s.value_mix == "source":
            keep = ctx.ws.take(self._SHARED, (nt, nv), self.dtype)
            ctx.shared[self._SHARED] = keep
        elif s.value_mix == "mix":
            first = ctx.shared.get(self._SHARED)
            if first is None or first.shape != (nt, nv):
                raise PartError("a layer that mixes values runs after the layer that is their source, "
                                "with values of the same width")
            mix = self.w["value_mix"].reshape(1)
        angles = self.rotary.angles(ctx) if self.rotary is not None else None
        kernels.qk_prepare(qkv, self.nq, self.nkv, self.dk, self.dv, float(s.eps),
                           self.w.get("q_norm.weight"), self.w.get("k_norm.weight"), angles, s.rot_dims,
                           mix, first, keep, meta.dest if writes_cache else None, kc, vc,
                           per_head=self.per_head)
        if not self._on_matrix_cores():
            o = ctx.ws.take("attention.o", (nt, self.nq * self.dv), self.dtype)
            kernels.attention_generic_dv(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen,
                                         self.nq, self.nkv, self.dk, self.dv, float(s.scale), s.window)
            return linear_delta(o, self.w["out.weight"], ctx.ws, "attention.delta"), None
        o = ctx.ws.take("attention.o", (nt, self.nq * self.dk), self.dtype)
        planner = self.step_planner()
        if ctx.all_single and planner is not None:
            plan = meta.plans.get(planner, {})
            kernels.attention_keys(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_kv_len,
                                   self.nq, self.nkv, self.dk, float(s.scale), s.window,
                                   units=plan.get("units"), seq_units=plan.get("seq_units"))
        else:
            kernels.attention_rows(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen,
                                   self.nq, self.nkv, self.dk, float(s.scale), s.window)
        w = self.out_wide if self.out_wide is not None else self.w["out.weight"]
        return linear_delta(o, w, ctx.ws, "attention.delta"), None


register_part("attention_normed", NormedAttention)


class SinkAttention(Part):
    """Softmax attention with key and value widths of their own, capped scores, a window and one
    more term in the softmax denominator (``SinkAttentionSpec``).

    One merged product gives [q | k | v | gate] (k and v only where the layer has keys and values of
    its own, the gate only where the heads are gated). Where the spec names a convolution, q, k and
    v pass it channel by channel (``kernels.causal_conv``, which keeps a sequence's last projected
    rows between steps). ``kernels.qk_rotate_store`` adds the biases where there is no convolution to
    take them, turns q and k and writes k and v to the paged cache; ``kernels.attention_sink`` reads
    the cache with scores, cap, sink, softmax and sums in float32 and applies the heads' gate; the
    output projection follows. A layer that borrows reads the lender's cache layer through its
    schedule entry and declares the same need."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if s.num_heads % s.num_kv_heads:
            raise PartError(f"{s.num_heads} heads do not divide into {s.num_kv_heads} kv heads")
        if not (2 <= s.key_dim <= 256 and s.key_dim % 2 == 0 and 1 <= s.value_dim <= 256):
            raise PartError(f"attention takes even key widths and value widths in [1, 256], not {s.key_dim} / {s.value_dim}")
        if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.key_dim or s.rot_style not in ("half", "interleaved"):
            raise PartError(f"{s.rot_dims} rotated coordinates ({s.rot_style!r}) do not fit heads of {s.key_dim}")
        if s.window is not None and s.window < 1:
            raise PartError(f"attention window must be >= 1, got {s.window}")
        if s.cache_window is not None and (s.cache_window < 0 or
                                           (s.cache_window > 0 and (s.window is None or s.cache_window < s.window))):
            raise PartError(f"a cache kept for {s.cache_window} tokens does not serve a window of {s.window}")
        if s.sink not in (None, "unit", "learned"):
            raise PartError(f"unknown sink {s.sink!r}")
        if s.softcap is not None and not s.softcap > 0:
            raise PartError(f"a score cap must be positive, got {s.softcap}")
        if s.conv_taps < 0 or (s.conv_taps and not s.own_kv):
            raise PartError("a convolution on q, k and v needs keys and values of the layer's own")
        self.spec, self.dtype = s, dtype
        self.nq, self.nkv, self.dk, self.dv = s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim
        self.qkv_width = self.nq * self.dk + (self.nkv * (self.dk + self.dv) if s.own_kv else 0)
        self.width = self.qkv_width + (self.nq * self.dv if s.out_gate else 0)
        self.rotary = None
        if s.rot_dims:
            from ..config.spec import PositionSpec
            self.rotary = build_part(PositionSpec(head_dim=s.rot_dims, theta=s.rot_base, style=s.rot_style,
                                                  ramp=s.rot_ramp, magnitude=s.rot_magnitude), dtype, device)

    def params(self):
        s = self.spec
        p = {"in.weight": Param((self.width, s.hidden), "matrix"),        # q, k, v, gate
             "out.weight": Param((s.hidden, self.nq * self.dv), "matrix")}
        if s.qkv_bias:
            p["in.bias"] = Param((self.qkv_width,), "vector")
        if s.conv_taps:
            p["conv.weight"] = Param((self.qkv_width, s.conv_taps), "vector")
        if s.sink == "learned":
            p["sink"] = Param((self.nq,), "vector", init="zero")
        return p

    # bfloat16 with a key width the matrix-core kernels take and values no wider than the keys: the
    # cache keeps value rows of the keys' width (the rest zero), so that the kernels for equal widths
    # serve prompts and single tokens, and the output projection reads the heads' rows through a copy
    # of its matrix with zero columns in the same places (as ``NormedAttention`` does). This depends on
    # the type and the two widths alone, which a layer shares with the readers of its cache. Everything
    # else (float32, other widths) runs the vector-ALU kernel on values of their own width.
    def _pads_values(self) -> bool:
        return self.dtype == torch.bfloat16 and self.dk % 32 == 0 and 32 <= self.dk <= 256 and self.dv <= self.dk

    def _on_matrix_cores(self) -> bool:
        # ... and rows of q that start on 16 bytes; a layer whose rows do not reads the padded cache
        # through the vector-ALU kernel
        return self._pads_values() and self.width % 8 == 0 and self.qkv_width % 8 == 0

    def step_planner(self):
        if self._on_matrix_cores() and kernels.keys_sink_fits(self.nq, self.nkv, self.dk):
            return KeyUnitPlanner(self.nkv)
        return None

    def bind(self, tensors):
        super().bind(tensors)
        self.out_wide = None
        if self._pads_values() and self.dv < self.dk and tensors["out.weight"].is_cuda:
            w = tensors["out.weight"]
            wide = torch.zeros(w.shape[0], self.nq, self.dk, dtype=w.dtype, device=w.device)
            wide[:, :, :self.dv] = w.view(w.shape[0], self.nq, self.dv)
            self.out_wide = wide.view(w.shape[0], self.nq * self.dk)

    def cache_need(self):
        s = self.spec
        # cache_window None: the layer's own window; 0: every token is kept; else that many
        window = s.window if s.cache_window is None else (s.cache_window or None)
        kv = KVNeed(self.nkv, self.dk, window, self.dk if self._pads_values() else self.dv)
        if s.conv_taps > 1:
            from ..cache.storage import StateNeed
            return [kv, StateNeed((s.conv_taps - 1, self.qkv_width), torch.float32)]
        return kv

    # with many rows the output projection can add itself to the residual stream (``into``)
    def can_add(self, nt: int) -> bool:
        w = self.out_wide if getattr(self, "out_wide", None) is not None else self.w["out.weight"]
        return adds_in_place(nt, w)

    def run(self, h, ctx, cache, layer, writes_cache=True, into=None):
        s, nt = self.spec, h.shape[0]
        if not s.own_kv and writes_cache:
            raise PartError("a layer without keys and values of its own runs on another layer's cache")
        proj = linear(h, self.w["in.weight"], ctx.ws.take("attention.in", (nt, self.width), self.dtype))
        kv_layer = layer[0] if isinstance(layer, (list, tuple)) else layer
        kc, vc, group = cache.layer_kv(kv_layer)
        meta = ctx.kv[group]
        bias = self.w.get("in.bias")
        if s.conv_taps:
            qkv = ctx.ws.take("attention.conv", (nt, self.qkv_width), self.dtype)
            kernels.causal_conv(proj, 0, self.qkv_width, self.w["conv.weight"], qkv,
                                cache.layer_state(layer[1]) if s.conv_taps > 1 else None, ctx.cu_q, ctx.slots,
                                ctx.max_qlen, bias_in=bias)
            bias = None
        else:
            qkv = proj[:, :self.qkv_width]
        angles = self.rotary.angles(ctx) if self.rotary is not None else None
        kernels.qk_rotate_store(qkv, self.nq, self.nkv, self.dk, self.dv, s.own_kv, bias, angles, s.rot_dims,
                                s.rot_style, meta.dest if (writes_cache and s.own_kv) else None, kc, vc)
        sink = self.w["sink"] if s.sink == "learned" else s.sink
        gate = proj[:, self.qkv_width:] if s.out_gate else None
        w = self.out_wide if self.out_wide is not None else self.w["out.weight"]
        if not self._on_matrix_cores():
            vd = self.dk if self._pads_values() else self.dv          # the width of the cache's value rows
            o = ctx.ws.take("attention.o", (nt, self.nq * vd), self.dtype)
            kernels.attention_sink(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen, self.nq,
                                   self.nkv, self.dk, vd, float(s.scale), s.window, s.softcap, sink, gate, self.dv)
            return linear_delta(o, w, ctx.ws, "attention.delta", into=into), None
        # matrix cores: scores and sums in float32, the softmax weights kept at 32 bits by three pieces
        o = ctx.ws.take("attention.o", (nt, self.nq * self.dk), self.dtype)
        planner = self.step_planner()
        # (the units of work are planned with the step's tables for the layer that owns the cache; a
        # reader whose lender has none takes the prompt kernel, which serves single tokens too)
        plan = meta.plans.get(planner) if planner is not None else None
        if ctx.all_single and plan:
            kernels.attention_keys_sink(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_kv_len, self.nq,
                                        self.nkv, self.dk, float(s.scale), s.window, s.softcap, sink, gate, self.dv,
                                        units=plan.get("units"), seq_units=plan.get("seq_units"))
        else:
            kernels.attention_rows_sink(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen, self.nq,
                                        self.nkv, self.dk, float(s.scale), s.window, s.softcap, sink, gate, self.dv)
        return linear_delta(o, w, ctx.ws, "attention.delta", into=into), None


register_part("attention_sink", SinkAttention)
