"""Mixers that keep a state of fixed size per sequence instead of a cache of keys.

``DiagonalRecurrence``: a gated linear recurrence per channel behind a short causal
convolution (the recurrent block of De et al., "Griffin: Mixing Gated Linear Recurrences with
Local Attention for Efficient Language Models"). ``GatedLinearAttention``: a matrix state per
head with a decay per key channel. Both walk a sequence's tokens in order in float32, so the
result does not depend on how the sequence was cut into steps; a step's products (the input
and output projections) are the framework's usual ones.
"""
from __future__ import annotations

import torch

from .. import kernels
from ..cache.storage import StateNeed
from ..weights.loader import Param
from .base import Part, PartError, register_part
from .linear import linear, linear_delta


class DiagonalRecurrence(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if s.channels < 1 or s.blocks < 1 or s.channels % s.blocks:
            raise PartError(f"{s.channels} channels do not divide into {s.blocks} blocks")
        if s.taps < 1:
            raise PartError(f"a convolution needs at least one tap, got {s.taps}")
        self.spec, self.dtype = s, dtype

    def params(self):
        s = self.spec
        C, bs = s.channels, s.channels // s.blocks
        return {"in.weight": Param((2 * C, s.hidden), "matrix"),       # y branch, then x branch
                "in.bias": Param((2 * C,), "vector"),
                "conv.weight": Param((C, s.taps), "vector"),
                "conv.bias": Param((C,), "vector"),
                "gates.weight": Param((2 * s.blocks, bs, bs), "matrix"),   # recurrence gate, then input gate
                "gates.bias": Param((2 * s.blocks, bs), "vector"),
                "lam": Param((C,), "vector"),
                "out.weight": Param((s.hidden, C), "matrix")}

    def cache_need(self):
        s = self.spec
        return [StateNeed((s.channels,), torch.float32), StateNeed((s.taps - 1, s.channels), torch.float32)]

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt, C = self.spec, h.shape[0], self.spec.channels
        state, conv_state = cache.layer_state(layer[0]), cache.layer_state(layer[1])
        yx = linear(h, self.w["in.weight"], ctx.ws.take("recurrence.in", (nt, 2 * C), self.dtype))
        a = ctx.ws.take("recurrence.a", (nt, C), torch.float32)
        b = ctx.ws.take("recurrence.b", (nt, C), torch.float32)
        bias = self.w["in.bias"]
        gates = kernels.rglru_gates
        args = ()
        if self.dtype == torch.bfloat16 and self.w["gates.weight"].dtype == torch.bfloat16 and \
                kernels.RGLRU_LIBRARY_ROWS <= nt <= 65535:
            gates, args = kernels.rglru_gates_split, (ctx.ws,)      # long steps: the library's batched product
        gates(yx, C, bias[C:], self.w["conv.weight"], self.w["conv.bias"], conv_state,
              self.w["gates.weight"], self.w["gates.bias"], self.w["lam"],
              float(s.decay_scale), ctx.cu_q, ctx.slots, a, b, *args)
        o = kernels.rglru_scan(yx, C, bias[:C], bias[C:], a, b, state, conv_state, ctx.cu_q, ctx.slots,
                               ctx.ws.take("recurrence.o", (nt, C), self.dtype), ctx.max_qlen,
                               ctx.ws.take("recurrence.s0", (ctx.batch, C), torch.float32))
        return linear_delta(o, self.w["out.weight"], ctx.ws, "recurrence.delta"), None


class GatedLinearAttention(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if not (s.key_dim >= 1 and s.value_dim >= 1 and s.rank >= 1 and s.num_heads >= 1):
            raise PartError(f"gated linear attention: heads {s.num_heads} of {s.key_dim} / {s.value_dim}, "
                            f"rank {s.rank}")
        if not s.tau > 0:
            raise PartError(f"gated linear attention: tau must be positive, got {s.tau}")
        self.spec, self.dtype = s, dtype
        self.width = 2 * s.num_heads * s.key_dim + 2 * s.num_heads * s.value_dim + s.rank

    def params(self):
        s = self.spec
        H, dk, dv = s.num_heads, s.key_dim, s.value_dim
        return {"in.weight": Param((self.width, s.hidden), "matrix"),     # q, k, v, gate, decay input
                "decay.weight": Param((H * dk, s.rank), "matrix"),
                "decay.bias": Param((H * dk,), "vector"),
                "norm.weight": Param((dv,), "vector", init="around_one"),
                "out.weight": Param((s.hidden, H * dv), "matrix")}

    def cache_need(self):
        s = self.spec
        return StateNeed((s.num_heads, s.key_dim, s.value_dim), torch.float32)

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt = self.spec, h.shape[0]
        H, dk, dv = s.num_heads, s.key_dim, s.value_dim
        proj = linear(h, self.w["in.weight"], ctx.ws.take("gla.in", (nt, self.width), self.dtype))
        o = kernels.gla_recurrent(proj, H, dk, dv, s.rank, self.w["decay.weight"], self.w["decay.bias"],
                                  float(s.tau), cache.layer_state(layer), ctx.cu_q, ctx.slots,
                                  ctx.ws.take("gla.o", (kernels.gla_row_parts(dk), nt, H, dv), torch.float32),
                                  ctx.ws.take("gla.alpha", (nt, H * dk), torch.float32))
        g = kernels.gla_out(o, proj, H, dk, dv, self.w["norm.weight"], float(s.eps),
                            ctx.ws.take("gla.gated", (nt, H * dv), self.dtype))
        return linear_delta(g, self.w["out.weight"], ctx.ws, "gla.delta"), None


class BonusRecurrence(Part):
    """The matrix-state recurrence with a bonus for the current token (``BonusRecurrenceSpec``).

    Its five inputs are token-shifted rows with a weight vector each; the previous token's row
    is the first of its two pieces of state, the heads' matrices the second. The kernels are
    those of ``GatedLinearAttention`` with the readout placed before the update (the recurrence
    walks a sequence's tokens in order in float32; decays and state never leave float32)."""
    graph_safe = True
    SHIFTS = 5          # r, k, v, gate, decay: the order of the rows of ``mu``

    def __init__(self, spec, dtype, device):
        s = spec
        if min(s.num_heads, s.head_dim, s.decay_rank) < 1:
            raise PartError(f"bonus recurrence: heads {s.num_heads} of {s.head_dim}, decay rank {s.decay_rank}")
        self.spec, self.dtype = s, dtype
        self.n = s.num_heads * s.head_dim

    def params(self):
        s, n = self.spec, self.n
        return {"mu": Param((self.SHIFTS * s.hidden,), "vector"),
                "rkvg.weight": Param((4 * n, s.hidden), "matrix"),      # r, k, v, gate: four blocks of rows
                "w1.weight": Param((s.decay_rank, s.hidden), "matrix"),
                "w2.weight": Param((n, s.decay_rank), "matrix"),
                "w0": Param((n,), "vector"),
                "bonus": Param((s.num_heads, s.head_dim), "vector"),
                "norm.weight": Param((n,), "vector", init="around_one"),
                "out.weight": Param((s.hidden, n), "matrix")}

    def cache_need(self):
        s = self.spec
        return [StateNeed((s.hidden,), torch.float32),
                StateNeed((s.num_heads, s.head_dim, s.head_dim), torch.float32)]

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt, n = self.spec, h.shape[0], self.n
        H, dk = s.num_heads, s.head_dim
        shift_state, state = cache.layer_state(layer[0]), cache.layer_state(layer[1])
        mixed = kernels.token_shift_multi(h, ctx.ws.take("bonus.mixed", (self.SHIFTS, nt, s.hidden), self.dtype),
                                          self.w["mu"].view(self.SHIFTS, s.hidden), shift_state, ctx.cu_q, ctx.slots)
        rkvg = ctx.ws.take("bonus.rkvg", (4, nt, n), self.dtype)
        w = self.w["rkvg.weight"].view(4, n, s.hidden)
        for i in range(4):
            linear(mixed[i], w[i], rkvg[i])
        low = linear(mixed[4], self.w["w1.weight"], ctx.ws.take("bonus.low", (nt, s.decay_rank), self.dtype))
        o = kernels.wkv_recurrent(rkvg, low, H, dk, dk, self.w["w2.weight"], self.w["w0"], self.w["bonus"], state,
                                  ctx.cu_q, ctx.slots,
                                  ctx.ws.take("bonus.o", (kernels.gla_row_parts(dk), nt, H, dk), torch.float32),
                                  ctx.ws.take("bonus.decay", (nt, n), torch.float32))
        g = kernels.head_norm_gate(o, rkvg[3], H, dk, self.w["norm.weight"], float(s.eps),
                                   ctx.ws.take("bonus.gated", (nt, n), self.dtype))
        return linear_delta(g, self.w["out.weight"], ctx.ws, "bonus.delta"), None


class DecayLinearAttention(Part):
    """Linear attention with one fixed decay per head and no softmax or denominator
    (``DecayLinearAttentionSpec``): S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t.

    One merged product gives [q | k | v | gate]. Options of the spec, each a kernel step of its
    own: an activation on q, k, v; a rotation of the first coordinates of every head of q and k
    (the keys go back into their rows); a scale on the keys, which the recurrence applies to
    the queries instead (the readout is linear in both); the norm of the readout per head or
    over all heads at once, with or without a weight; the gate's activation. The recurrence is
    the kernel of ``GatedLinearAttention`` with the head's constant in place of a decay per
    key channel and token: state, decays and readout stay float32, tokens are walked in order,
    so a cut of the sequence changes nothing."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if min(s.num_heads, s.key_dim, s.value_dim) < 1:
            raise PartError(f"linear attention: {s.num_heads} heads of {s.key_dim} / {s.value_dim}")
        if len(s.decays) != s.num_heads:
            raise PartError(f"linear attention: {len(s.decays)} decays for {s.num_heads} heads")
        if any(not 0.0 <= float(a) <= 1.0 for a in s.decays):
            raise PartError(f"linear attention: decays must lie in [0, 1], got {tuple(s.decays)}")
        if s.input_activation not in (None, "silu") or s.gate_activation not in ("silu", "sigmoid"):
            raise PartError(f"linear attention: activations {s.input_activation!r} / {s.gate_activation!r}")
        if s.head_norm not in ("per_head", "all_heads"):
            raise PartError(f"linear attention: unknown head_norm {s.head_norm!r}")
        if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.key_dim:
            raise PartError(f"{s.rot_dims} rotated coordinates do not fit heads of {s.key_dim}")
        self.spec, self.dtype = s, dtype
        self.nk, self.nv = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        self.width = 2 * self.nk + 2 * self.nv
        self.decays = torch.tensor([float(a) for a in s.decays], dtype=torch.float32, device=device)
        self.rotary = None
        if s.rot_dims:
            from ..config.spec import PositionSpec
            from .base import build_part
            self.rotary = build_part(PositionSpec(head_dim=s.rot_dims, theta=s.rot_base, style="half",
                                                  scaling=s.rot_scaling), dtype, device)

    def params(self):
        s = self.spec
        p = {"in.weight": Param((self.width, s.hidden), "matrix"),       # q, k, v, gate
             "out.weight": Param((s.hidden, self.nv), "matrix")}
        if s.norm_weight:
            n = self.nv if s.head_norm == "all_heads" else s.value_dim
            p["norm.weight"] = Param((n,), "vector", init="around_one")
        return p

    def cache_need(self):
        s = self.spec
        return StateNeed((s.num_heads, s.key_dim, s.value_dim), torch.float32)

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt = self.spec, h.shape[0]
        H, dk, dv = s.num_heads, s.key_dim, s.value_dim
        proj = linear(h, self.w["in.weight"], ctx.ws.take("decay_attention.in", (nt, self.width), self.dtype))
        qkv = proj[:, :2 * self.nk + self.nv]
        if s.input_activation is not None:
            kernels.activation(qkv, qkv, s.input_activation)
        if self.rotary is not None:
            kernels.qk_prepare(qkv, H, H, dk, dv, float(s.eps), None, None, self.rotary.angles(ctx), s.rot_dims,
                               k_inplace=True)
        o = kernels.decay_recurrent(proj, 0, self.nk, 2 * self.nk, H, dk, dv, self.decays, float(s.key_scale),
                                    cache.layer_state(layer), ctx.cu_q, ctx.slots,
                                    ctx.ws.take("decay_attention.o", (kernels.gla_row_parts(dk), nt, H, dv),
                                                torch.float32))
        gate = proj[:, 2 * self.nk + self.nv:]
        gated = ctx.ws.take("decay_attention.gated", (nt, self.nv), self.dtype)
        if s.head_norm == "all_heads":
            kernels.head_norm_gate(o.view(o.shape[0], nt, 1, self.nv), gate, 1, self.nv, self.w.get("norm.weight"),
                                   float(s.eps), gated, s.gate_activation)
        else:
            kernels.head_norm_gate(o, gate, H, dv, self.w.get("norm.weight"), float(s.eps), gated,
                                   s.gate_activation)
        return linear_delta(gated, self.w["out.weight"], ctx.ws, "decay_attention.delta"), None


class StateSpace(Part):
    """The selective state-space mixer with a scalar decay per head (``StateSpaceSpec``).

    One product gives [z | x | B | C | dt]; ``kernels.causal_conv`` runs the convolution with bias and
    silu over [x | B | C] (its memory is the second piece of state); ``kernels.ssm_steps`` forms step
    sizes and decays of every (token, head) in float32; the recurrence is the kernel of
    ``GatedLinearAttention`` with q = C, k = B, v = x, the heads of a group reading the same B and C,
    one decay per (token, head) and the step size as a factor on the key, so state, decays and
    readout stay float32 and tokens are walked in order; ``kernels.gated_group_norm`` adds D x, gates
    with silu(z) and norms the parts of the row."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        s = spec
        if min(s.num_heads, s.head_dim, s.state, s.groups, s.taps, s.norm_groups) < 1:
            raise PartError(f"state space: {s.num_heads} heads of {s.head_dim}, state {s.state}, {s.groups} groups, "
                            f"{s.taps} taps, {s.norm_groups} norm parts")
        if s.num_heads % s.groups or (s.num_heads * s.head_dim) % s.norm_groups:
            raise PartError(f"state space: {s.num_heads} heads of {s.head_dim} do not divide into {s.groups} "
                            f"groups / {s.norm_groups} norm parts")
        self.spec, self.dtype = s, dtype
        self.inner = s.num_heads * s.head_dim
        self.gn = s.groups * s.state
        self.conv_width = self.inner + 2 * self.gn
        self.width = self.inner + self.conv_width + s.num_heads

    def params(self):
        s = self.spec
        H = s.num_heads
        return {"in.weight": Param((self.width, s.hidden), "matrix"),       # z, x, B, C, dt
                "conv.weight": Param((self.conv_width, s.taps), "vector"),
                "conv.bias": Param((self.conv_width,), "vector"),
                "dt_bias": Param((H,), "vector", init="zero"),
                "A_log": Param((H,), "vector", init="zero"),
                "D": Param((H,), "vector", init="around_one"),
                "norm.weight": Param((self.inner,), "vector", init="around_one"),
                "out.weight": Param((s.hidden, self.inner), "matrix")}

    def cache_need(self):
        s = self.spec
        need = [StateNeed((s.num_heads, s.state, s.head_dim), torch.float32)]
        if s.taps > 1:
            need.append(StateNeed((s.taps - 1, self.conv_width), torch.float32))
        return need

    def run(self, h, ctx, cache, layer, writes_cache=True):
        s, nt = self.spec, h.shape[0]
        H, P, N = s.num_heads, s.head_dim, s.state
        proj = linear(h, self.w["in.weight"], ctx.ws.take("state_space.in", (nt, self.width), self.dtype))
        xbc = ctx.ws.take("state_space.xbc", (nt, self.conv_width), self.dtype)
        kernels.causal_conv(proj, self.inner, self.conv_width, self.w["conv.weight"], xbc,
                            cache.layer_state(layer[1]) if s.taps > 1 else None, ctx.cu_q, ctx.slots,
                            ctx.max_qlen, bias_out=self.w["conv.bias"],
                            activation="silu")
        dt = ctx.ws.take("state_space.dt", (nt, H), torch.float32)
        decay = ctx.ws.take("state_space.decay", (nt, H), torch.float32)
        kernels.ssm_steps(proj, self.inner + self.conv_width, H, self.w["dt_bias"], self.w["A_log"], dt, decay)
        o = kernels.ssm_recurrent(xbc, 0, self.inner, self.inner + self.gn, H, s.groups, N, P, decay, dt,
                                  cache.layer_state(layer[0]), ctx.cu_q, ctx.slots,
                                  ctx.ws.take("state_space.o", (kernels.gla_row_parts(N), nt, H, P), torch.float32))
        y = kernels.gated_group_norm(o.view(o.shape[0], nt, self.inner), proj, 0, self.w["norm.weight"], float(s.eps),
                                     s.norm_groups, ctx.ws.take("state_space.y", (nt, self.inner), self.dtype),
                                     x=xbc, x_off=0, skip=self.w["D"], head_dim=P)
        return linear_delta(y, self.w["out.weight"], ctx.ws, "state_space.delta"), None


register_part("state_space", StateSpace)
register_part("diagonal_recurrence", DiagonalRecurrence)
register_part("decay_linear_attention", DecayLinearAttention)
register_part("bonus_recurrence", BonusRecurrence)
register_part("gated_linear_attention", GatedLinearAttention)
