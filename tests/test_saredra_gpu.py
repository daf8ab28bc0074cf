"""The Saredra decoder on the GPU against the plain implementation in ``plain_saredra``.

Each mechanism alone (its kernels against the plain function, with cache and state carried over
cuts), then the engine: layers, whole prompts, portions, token-by-token decoding, unequal
batches, slots and pages used again, recorded steps, far keys and keys at the borders of pages
and windows, long decoding, greedy generation, the replayer and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_saredra as P
import saredra_util as U

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def _t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def _bf(a, dtype="bfloat16"):
    from plain_llama import round_bf16
    a = np.asarray(a, dtype=np.float64)
    return round_bf16(a) if dtype == "bfloat16" else a.astype(np.float32).astype(np.float64)


def _np(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def _close(got, want, dtype, what="", scale=1.0):
    tol = (3e-5 if dtype == "float32" else 2.5e-2) * scale
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), what


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("d", [72, 90, 1024])
@pytest.mark.parametrize("n", [1, 2, 3])
def test_weighted_sum_of_branches(d, n):
    from transformer_amd import kernels as K
    rng = np.random.default_rng(d + n)
    for nt in (1, 7, 130):
        deltas = [rng.standard_normal((1 + (i + nt) % 3, nt, d)).astype(np.float32) for i in range(n)]
        deltas[0] = deltas[0][0]                                   # one without planes
        scales = [1.2, 0.9, -0.5][:n]
        out = torch.empty(nt, d, device=DEV)
        K.weighted_sum([_t(x) for x in deltas], scales, out)
        want = sum(s * (x.astype(np.float64).sum(0) if x.ndim == 3 else x) for s, x in zip(scales, deltas))
        np.testing.assert_allclose(_np(out), want, atol=1e-5)


@pytest.mark.parametrize("geom", [(6, 2, 3, 2), (8, 2, 2, 1), (4, 4, 1, 1), (1, 1, 1, 1), (9, 4, 3, 3), (64, 6, 8, 3), (12, 3, 12, 3),
                                  (10, 5, 5, 5)])
def test_routing_in_groups(geom):
    from transformer_amd import kernels
    E, top, groups, keep = geom
    rng = np.random.default_rng(E * 10 + top)
    nt = 60
    z = (2.0 * rng.standard_normal((nt, E + 2))).astype(np.float32)            # more columns than experts
    chosen = torch.empty(nt, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(nt, top, device=DEV)
    kernels.moe_route(_t(z), E, top, chosen, weight, "softmax", False, groups=groups, keep_groups=keep)
    s = np.exp(z[:, :E].astype(np.float64))
    s /= s.sum(1, keepdims=True)
    got_c, got_w = chosen.cpu().numpy(), _np(weight)
    differs = False
    for t in range(nt):
        want = P.route(s[t], top, groups, keep)
        assert list(got_c[t]) == list(want), (t, got_c[t], want)
        np.testing.assert_allclose(got_w[t], s[t][want], atol=1e-6)            # the scores themselves, not renormalised
        differs = differs or sorted(want) != sorted(P.route(s[t], top))
    if keep < groups and E // groups > 1 and (keep == 1 or top > keep):
        assert differs                                                       # the groups changed somebody's choice


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(6, 2, 24, 72, 3, 2), (4, 4, 16, 72, 1, 1), (1, 1, 32, 64, 1, 1), (9, 4, 10, 90, 3, 3),
                                  (12, 3, 48, 328, 4, 2), (8, 2, 256, 1024, 4, 2)])
def test_routed_gated_experts_part(dtype, geom):
    """The routed feed-forward as the block runs it (scores, groups, ordering, both products, the
    gate, the weighted sum back) against the plain function."""
    from transformer_amd.config.spec import RoutedMLPSpec
    from transformer_amd.parts.base import build_part
    from transformer_amd.parts.linear import Workspace
    E, top, ff, d, gc, gk = geom
    rng = np.random.default_rng(E + top + ff)
    m = {"router": {"experts": E, "top": top, "groups": {"count": gc, "keep": gk}}, "expert": {"ff": ff}}
    shapes = {"router": (E, d)}
    for e in range(E):
        shapes.update({f"e{e}.gate": (ff, d), f"e{e}.up": (ff, d), f"e{e}.down": (d, ff)})
    w = {n: _bf((4.0 if n == "router" else 2.0) * rng.standard_normal(s) / np.sqrt(s[-1]), dtype) for n, s in shapes.items()}
    spec = RoutedMLPSpec(hidden=d, experts=E, top=top, intermediate=ff, activation="silu", score="softmax",
                         renormalize=False, weight_on="output", shared_intermediate=None, shared_gate=False, form="glu",
                         groups=gc, keep_groups=gk)
    part = build_part(spec, TD[dtype], DEV)
    mat = lambda a: _t(a, TD[dtype])
    part.bind({"router.weight": mat(w["router"]),
               "experts.gate_up.weight": mat(np.concatenate([w[f"e{e}.{n}"] for e in range(E) for n in ("gate", "up")])),
               "experts.down.weight": mat(np.concatenate([w[f"e{e}.down"] for e in range(E)]))})

    class Ctx:
        ws, dump = Workspace(DEV), None
    for nt in (1, 9, 150):
        h = _bf(rng.standard_normal((nt, d)), dtype)
        chosen = {}
        Ctx.dump = lambda name, t: chosen.__setitem__(name, t.cpu().numpy().astype(np.int64))
        delta, bias = part.run(mat(h), Ctx)
        assert bias is None
        want, _ = P.moe(h, w, "", m, forced=None if dtype == "float32" else chosen["experts"], slack=U.SLACK)
        _close(_np(delta), want, dtype, f"{nt} rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(40, 4, True, "silu"), (7, 1, False, None), (300, 2, True, None), (33, 7, False, "silu"),
                                  (1, 3, True, "silu"), (20, 9, True, None), (70, 8, False, "silu")])
def test_short_convolution_over_cuts(dtype, geom):
    """Three sequences of unequal lengths in slots that held something else, fed in cuts of many,
    one, two and two tokens: the convolution's memory carries the last inputs (with the
    projection's bias) from cut to cut; the inputs are a range of columns of wider rows."""
    from transformer_amd import kernels as K
    C, taps, in_bias, act = geom
    rng = np.random.default_rng(C * 10 + taps)
    lens, off, wide = [37, 1, 12], 5, C + 9
    seqs = [_bf(rng.standard_normal((L + 5, wide)), dtype) for L in lens]
    w = rng.standard_normal((C, taps)).astype(np.float32).astype(np.float64)
    bi = rng.standard_normal(C).astype(np.float32).astype(np.float64) if in_bias else None
    bo = rng.standard_normal(C).astype(np.float32).astype(np.float64)
    state = torch.full((5, taps - 1, C), 3.0, device=DEV) if taps > 1 else None      # one tap: no memory
    slots = [3, 0, 4]
    if taps > 1:
        for s in slots:
            state[s] = 0.0
    got, done = [[] for _ in lens], [0] * len(lens)
    for part in (lambda L: L, lambda L: 1, lambda L: 2, lambda L: 2):
        rows = [s[a:a + part(L)] for s, L, a in zip(seqs, lens, done)]
        x = _t(np.concatenate(rows), TD[dtype])
        nt = x.shape[0]
        cu = _t(np.concatenate([[0], np.cumsum([len(r) for r in rows])]), torch.int32)
        out = torch.empty(nt, C, dtype=TD[dtype], device=DEV)
        K.causal_conv(x, off, C, _t(w), out, state, cu, _t(slots, torch.int32), max(len(r) for r in rows),
                      bias_in=None if bi is None else _t(bi), bias_out=_t(bo), activation=act)
        at = 0
        for i, r in enumerate(rows):
            got[i].append(_np(out[at:at + len(r)]))
            at += len(r)
            done[i] += len(r)
    for i, s in enumerate(seqs):
        u = s[:, off:off + C] + (0.0 if bi is None else bi)
        want = P.causal_conv(u, w, bo)
        if act == "silu":
            want = P.silu(want)
        _close(np.concatenate(got[i]), want, dtype, f"sequence {i}")
    if taps > 1:
        assert float(state[1].min()) == 3.0 and float(state[2].max()) == 3.0    # slots of others stay as they are
        np.testing.assert_allclose(_np(state[3]), (seqs[0][:, off:off + C] + (0.0 if bi is None else bi))[-(taps - 1):], atol=1e-6)


def _selectors(sizes):
    """Matrices that cut consecutive column ranges of the given sizes out of a row."""
    total, at, out = sum(sizes), 0, []
    for n in sizes:
        m = np.zeros((n, total))
        m[np.arange(n), at + np.arange(n)] = 1.0
        out.append(m)
        at += n
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(6, 2, 20, 12, 8, (4.0, 64, 8.0, 1.0), 37, 5.0, "learned"), (4, 4, 16, 24, 0, None, None, None, "unit"),
                                  (1, 1, 16, 16, 16, None, 64, 2.0, None), (5, 5, 6, 11, 6, None, 65, None, "learned"),
                                  (2, 1, 34, 6, 34, (3.0, 40, 6.0, 2.0), 1, 9.0, "unit"), (4, 1, 8, 40, 2, None, 129, 30.0, "learned"),
                                  (8, 2, 128, 64, 64, (2.0, 512, 16.0, 1.0), 100, 50.0, "unit")])
def test_capped_sunk_softmax_pieces(dtype, geom):
    """Biases, the rotation of neighbouring pairs with slowed frequencies and a magnitude, keys and
    values into shuffled pages that held NaN, capped scores, the window, both kinds of sink and the
    heads' gate; a prompt in two portions, two single tokens and another portion, against the plain
    functions."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    from transformer_amd.parts.position import ramp_frequencies
    H, G, dk, dv, rot, scaling, window, cap, sink = geom
    rng = np.random.default_rng(H * 7 + dk)
    T, scale, base = 150, 0.21, 500.0
    cols = (H + G) * dk + G * dv
    rows = _bf(rng.standard_normal((T, cols)), dtype)
    gate = _bf(rng.standard_normal((T, H * dv + 3)), dtype)
    bias = rng.standard_normal(cols).astype(np.float32).astype(np.float64)
    rotd, mag = None, 1.0
    if rot:
        rotd = {"dims": rot, "base": base}
        if scaling:
            rotd["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        f, mag = P.rotation_frequencies(rotd)
        if scaling:
            np.testing.assert_allclose(ramp_frequencies(rot, base, scaling), f, rtol=1e-12)
    sinks = rng.standard_normal(H) * 2.0
    u = rows + bias
    q = P.rotate_pairs(u[:, :H * dk].reshape(T, H, dk), np.arange(T), rotd)
    k = P.rotate_pairs(u[:, H * dk:(H + G) * dk].reshape(T, G, dk), np.arange(T), rotd)
    v = u[:, (H + G) * dk:].reshape(T, G, dv)
    want = P.windowed_softmax_attention(_bf(q, dtype), _bf(k, dtype), _bf(v, dtype), scale, cap, window,
                                        None if sink is None else np.zeros(H) if sink == "unit" else sinks)
    want = want.reshape(T, H * dv) * P.sigmoid(gate[:, :H * dv])
    kc = torch.full((9, G, PAGE, dk), float("nan"), dtype=TD[dtype], device=DEV)
    vc = torch.full((9, G, dv, PAGE), float("nan"), dtype=TD[dtype], device=DEV)
    pages = np.array([7, 2, 5])
    inv = _t(P.rotation_frequencies(rotd)[0]) if rot else None
    got, at = [], 0
    for n in (70, 58, 1, 1, 20):
        p = np.arange(at, at + n)
        qkv = _t(rows[p], TD[dtype])
        angles = K.rope_table(_t(p, torch.int32), inv, torch.empty(n, rot // 2, 2, device=DEV), mag) if rot else None
        dest = _t(pages[p // PAGE] * PAGE + p % PAGE, torch.int32)
        K.qk_rotate_store(qkv, H, G, dk, dv, True, _t(bias), angles, rot, "interleaved", dest, kc, vc)
        o = torch.empty(n, H * dv, dtype=TD[dtype], device=DEV)
        K.attention_sink(qkv, o, kc, vc, _t([pages], torch.int32), _t([0, n], torch.int32), _t([at], torch.int32), n,
                         H, G, dk, dv, scale, window, cap, _t(sinks) if sink == "learned" else sink,
                         _t(gate[p], TD[dtype]))
        got.append(_np(o))
        at += n
    _close(np.concatenate(got), want, dtype, scale=1.5)


@pytest.mark.parametrize("exact", [True, False])
@pytest.mark.parametrize("geom", [(8, 2, 128, 64, 64, (2.0, 512, 16.0, 1.0), 100, 50.0, "unit", True),
                                  (4, 4, 32, 32, 0, None, None, None, "learned", False),
                                  (16, 4, 64, 64, 32, None, 129, 30.0, "learned", True),
                                  (2, 1, 96, 40, 96, (3.0, 40, 6.0, 2.0), 64, 3.0, None, True),
                                  (6, 1, 160, 8, 10, None, 1, 9.0, "unit", False),
                                  (64, 2, 64, 64, 64, None, 200, 20.0, "learned", True)])
def test_capped_sunk_softmax_on_matrix_cores(geom, exact):
    """The same on the matrix-core kernels (bfloat16, value rows of the cache as wide as the keys, the
    rest zero): prompts through the kernel that reads pages directly and the one that shares them
    through LDS, single tokens through the kernel of four waves and the merge, with a page table
    wider than needed; with the weights kept at 32 bits the result is as close as the vector kernel's."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    H, G, dk, dv, rot, scaling, window, cap, sink, gated = geom
    dtype = "bfloat16"
    rng = np.random.default_rng(H * 7 + dk)
    T, scale, base = 600, 0.21 * (32 / dk) ** 0.5, 500.0
    cols = (H + G) * dk + G * dv
    rows = _bf(rng.standard_normal((T, cols)), dtype)
    gate = _bf(rng.standard_normal((T, H * dv + 8)), dtype)
    rotd, mag = None, 1.0
    if rot:
        rotd = {"dims": rot, "base": base}
        if scaling:
            rotd["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
        mag = P.rotation_frequencies(rotd)[1]
    sinks = rng.standard_normal(H) * 2.0
    q = P.rotate_pairs(rows[:, :H * dk].reshape(T, H, dk), np.arange(T), rotd)
    k = P.rotate_pairs(rows[:, H * dk:(H + G) * dk].reshape(T, G, dk), np.arange(T), rotd)
    v = rows[:, (H + G) * dk:].reshape(T, G, dv)
    want = P.windowed_softmax_attention(_bf(q, dtype), _bf(k, dtype), v, scale, cap, window,
                                        None if sink is None else np.zeros(H) if sink == "unit" else sinks)
    want = want.reshape(T, H * dv)
    if gated:
        want = want * P.sigmoid(gate[:, :H * dv])
    kc = torch.full((12, G, PAGE, dk), float("nan"), dtype=TD[dtype], device=DEV)
    vc = torch.full((12, G, dk, PAGE), float("nan"), dtype=TD[dtype], device=DEV)
    pages = np.array([7, 2, 5, 11, 0, 9, 4, 1, 3, 10, 0, 0])              # ten pages of a table of twelve
    inv = _t(P.rotation_frequencies(rotd)[0]) if rot else None
    got, at = [], 0
    for n, lds in ((70, 0), (300, 1), (1, None), (1, 0), (28, "vector"), (1, None), (199, 0)):
        p = np.arange(at, at + n)
        qkv = _t(rows[p], TD[dtype])
        angles = K.rope_table(_t(p, torch.int32), inv, torch.empty(n, rot // 2, 2, device=DEV), mag) if rot else None
        dest = _t(pages[p // PAGE] * PAGE + p % PAGE, torch.int32)
        K.qk_rotate_store(qkv, H, G, dk, dv, True, None, angles, rot, "interleaved", dest, kc, vc)
        o = torch.empty(n, H * dk, dtype=TD[dtype], device=DEV)
        args = (qkv, o, kc, vc, _t([pages], torch.int32), _t([0, n], torch.int32), _t([at], torch.int32))
        opts = (H, G, dk, scale, window, cap, _t(sinks) if sink == "learned" else sink, _t(gate[p], TD[dtype]) if gated else None, dv)
        if lds is None:
            K.attention_keys_sink(*args, at + 1, *opts, exact=exact)
        elif lds == "vector":                # the vector kernel over the padded cache: the gate's rows keep their width
            K.attention_sink(*args, n, H, G, dk, dk, scale, window, cap, opts[6], opts[7], dv)
        else:
            K.attention_rows_sink(*args, n, *opts, exact=exact, through_lds=lds)
        o = _np(o).reshape(n, H, dk)
        assert np.all(o[:, :, dv:] == 0.0)                                   # the padding of the values stays zero
        got.append(o[:, :, :dv].reshape(n, H * dv))
        at += n
    _close(np.concatenate(got), want, dtype, scale=1.5 if exact else 3.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("where", ["prompt", "decode"])
@pytest.mark.parametrize("mark,window", [(0, None), (3, None), (63, None), (64, None), (127, None), (128, None), (298, None),
                                         (200, 100), (199, 100), (236, 64), (235, 64), (171, 129), (170, 129), (299, 1), (298, 1)])
def test_one_key_stands_out(where, dtype, mark, window):
    """The last query points at ONE earlier key (the first token, hundreds back, the last and the
    first of a page, the first key inside a window and the last one outside): its score stands out
    under the cap, so the result is that key's value where the window holds it, and something else
    where it does not. The energy sits in coordinates that do not rotate."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    H, G, dk, dv, rot, T = 4, 2, 32, 24, 8, 300
    rng = np.random.default_rng(mark)
    q, k = 0.05 * rng.standard_normal((T, H * dk)), 0.05 * rng.standard_normal((T, G * dk))
    v = _bf(rng.standard_normal((T, G * dv)), dtype)
    k.reshape(T, G, dk)[mark, :, rot:rot + 4] = 3.0
    q.reshape(T, H, dk)[T - 1, :, rot:rot + 4] = 3.0
    rows = _bf(np.concatenate([q, k, v], 1), dtype)
    pages = np.array([4, 1, 3, 0, 5])
    kc = torch.full((6, G, PAGE, dk), float("nan"), dtype=TD[dtype], device=DEV)
    vc = torch.full((6, G, dv, PAGE), float("nan"), dtype=TD[dtype], device=DEV)
    inv = _t(100.0 ** (-2.0 * np.arange(rot // 2) / rot))
    nq = 1 if where == "decode" else 45
    for p in (np.arange(0, T - nq), np.arange(T - nq, T)):
        qkv = _t(rows[p], TD[dtype])
        angles = K.rope_table(_t(p, torch.int32), inv, torch.empty(len(p), rot // 2, 2, device=DEV))
        dest = _t(pages[p // PAGE] * PAGE + p % PAGE, torch.int32)
        K.qk_rotate_store(qkv, H, G, dk, dv, True, None, angles, rot, "interleaved", dest, kc, vc)
    o = torch.empty(nq, H * dv, dtype=TD[dtype], device=DEV)
    K.attention_sink(qkv, o, kc, vc, _t([pages], torch.int32), _t([0, nq], torch.int32), _t([T - nq], torch.int32),
                     nq, H, G, dk, dv, 1.0, window, 30.0, "unit")           # score 36 under a cap of 30: 25.0
    marked = np.repeat(v[mark].reshape(G, dv), H // G, axis=0).reshape(-1)
    seen = window is None or T - 1 - mark < window
    err = np.abs(_np(o[-1]) - marked).max()
    if seen:
        assert err < (1e-3 if dtype == "float32" else 2e-2)
    else:
        assert err > 0.5


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_takes_its_share(dtype):
    """One key per query (a window of 1) with score 0: a unit sink halves the value, a learned sink s
    leaves 1 / (1 + exp(s)) of it, no sink leaves all."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    H, G, dk, dv, T = 3, 1, 8, 5, 70
    rng = np.random.default_rng(0)
    v = _bf(rng.standard_normal((T, G * dv)), dtype)
    rows = np.concatenate([np.zeros((T, (H + G) * dk)), v], 1)
    kc = torch.zeros((2, G, PAGE, dk), dtype=TD[dtype], device=DEV)
    vc = torch.zeros((2, G, dv, PAGE), dtype=TD[dtype], device=DEV)
    qkv = _t(rows, TD[dtype])
    K.qk_rotate_store(qkv, H, G, dk, dv, True, None, None, 0, "interleaved", _t(np.arange(T), torch.int32), kc, vc)
    sinks = np.array([-30.0, 0.7, 4.0])
    for sink, share in ((None, np.ones(H)), ("unit", np.full(H, 0.5)), (_t(sinks), 1.0 / (1.0 + np.exp(sinks)))):
        o = torch.empty(T, H * dv, dtype=TD[dtype], device=DEV)
        K.attention_sink(qkv, o, kc, vc, _t([[0, 1]], torch.int32), _t([0, T], torch.int32), _t([0], torch.int32), T,
                         H, G, dk, dv, 0.3, 1, 5.0, sink)
        want = (v[:, None, :] * share[None, :, None]).reshape(T, H * dv)
        _close(_np(o), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(4, 12, 10, 2, 3), (1, 64, 16, 1, 1), (5, 7, 33, 1, 5), (4, 6, 40, 4, 2), (16, 64, 64, 2, 4),
                                  (3, 8, 6, 3, 1), (8, 32, 128, 8, 8), (6, 80, 24, 3, 2), (32, 128, 16, 4, 1)])
def test_state_space_pieces(dtype, geom):
    """Step sizes and decays, the recurrence with the state carried over cuts of many, one and two
    tokens, the skip, the gate before the norm and the norm in parts; three sequences of unequal
    lengths in slots that held something else; heads of a group reading the same B and C."""
    from transformer_amd import kernels as K
    H, Pd, N, G, ng = geom
    rng = np.random.default_rng(H * 100 + N)
    lens, eps = [37, 1, 12], 1e-5
    inner, gn = H * Pd, G * N
    seqs = [_bf(rng.standard_normal((L + 5, inner + 2 * gn)), dtype) for L in lens]       # x, B, C behind the convolution
    zdt = [_bf(rng.standard_normal((L + 5, inner + H + 2)), dtype) for L in lens]         # z, then dt
    dt_bias, a_log, D = rng.uniform(-3, 1, H), rng.uniform(-2, 1, H), rng.standard_normal(H)
    if H >= 3:
        a_log[0], dt_bias[1] = -30.0, 8.0                                                  # a decay of 1; a head that forgets fast
    nw = 1 + 0.2 * rng.standard_normal(inner)

    def plain_one(rows, zd):
        T = len(rows)
        dt = P.softplus(zd[:, inner:inner + H] + dt_bias)
        x = rows[:, :inner].reshape(T, H, Pd)
        B, C = rows[:, inner:inner + gn].reshape(T, G, N), rows[:, inner + gn:].reshape(T, G, N)
        y, _ = P.selective_scan(x, B, C, dt, a_log, D, G)
        if T <= 20:
            np.testing.assert_allclose(y, P.selective_scan_sum(x, B, C, dt, a_log, D, G), atol=1e-9)
        y = y.reshape(T, inner) * P.silu(zd[:, :inner])
        return P.grouped_unit_rms(y, ng, eps) * nw
    state = torch.full((5, H, N, Pd), 3.0, device=DEV)
    slots = [3, 0, 4]
    for s in slots:
        state[s] = 0.0
    got, done = [[] for _ in lens], [0] * len(lens)
    f32 = lambda a: _t(np.asarray(a, dtype=np.float32))
    for part in (lambda L: L, lambda L: 1, lambda L: 2, lambda L: 2):
        rows = [s[a:a + part(L)] for s, L, a in zip(seqs, lens, done)]
        xbc = _t(np.concatenate(rows), TD[dtype])
        zd = _t(np.concatenate([z[a:a + part(L)] for z, L, a in zip(zdt, lens, done)]), TD[dtype])
        nt = xbc.shape[0]
        cu = _t(np.concatenate([[0], np.cumsum([len(r) for r in rows])]), torch.int32)
        dt, decay = torch.empty(nt, H, device=DEV), torch.empty(nt, H, device=DEV)
        K.ssm_steps(zd, inner, H, f32(dt_bias), f32(a_log), dt, decay)
        o = torch.empty(K.gla_row_parts(N), nt, H, Pd, device=DEV)
        K.ssm_recurrent(xbc, 0, inner, inner + gn, H, G, N, Pd, decay, dt, state, cu, _t(slots, torch.int32), o)
        out = torch.empty(nt, inner, dtype=TD[dtype], device=DEV)
        K.gated_group_norm(o.view(o.shape[0], nt, inner), zd, 0, f32(nw), eps, ng, out, x=xbc, x_off=0, skip=f32(D), head_dim=Pd)
        at = 0
        for i, r in enumerate(rows):
            got[i].append(_np(out[at:at + len(r)]))
            at += len(r)
            done[i] += len(r)
    for i, s in enumerate(seqs):
        want = plain_one(s, zdt[i])
        _close(np.concatenate(got[i]), want, dtype, f"sequence {i}", scale=3.0)
    assert float(state[1].min()) == 3.0 and float(state[2].max()) == 3.0    # slots of others stay as they are


@pytest.mark.parametrize("where", ["prompt", "decode"])
def test_a_far_token_in_the_state(where):
    """Head 0 never forgets (its decay is 1 to float32), head 1 forgets at once, head 2 fades: a token
    497 steps back shows in head 0's readout as on the first day, not at all in head 1's, faded in
    head 2's."""
    from transformer_amd import kernels as K
    H, Pd, N, T, far = 3, 4, 4, 500, 2
    rng = np.random.default_rng(5)
    x = 0.01 * rng.standard_normal((T, H * Pd))
    B, C = np.zeros((T, N)), np.zeros((T, N))
    B[:, 1], C[:, 1] = 0.1, 0.1
    B[far, 0], C[T - 1, 0] = 8.0, 8.0
    x[far] = rng.standard_normal(H * Pd)
    rows = np.concatenate([x, B, C], 1)
    a_log = np.array([-40.0, 5.0, np.log(0.01)])
    dt = np.ones((T, H))
    decay = np.exp(-np.exp(a_log))[None, :] * np.ones((T, 1))
    want, _ = P.selective_scan(x.reshape(T, H, Pd), B.reshape(T, 1, N), C.reshape(T, 1, N), dt, a_log, np.zeros(H), 1)
    state = torch.zeros((1, H, N, Pd), device=DEV)
    nq = 1 if where == "decode" else 33
    f32 = lambda a: _t(np.asarray(a, dtype=np.float32))
    for lo, hi in ((0, T - nq), (T - nq, T)):
        xbc = f32(rows[lo:hi])
        o = torch.empty(K.gla_row_parts(N), hi - lo, H, Pd, device=DEV)
        K.ssm_recurrent(xbc, 0, H * Pd, H * Pd + N, H, 1, N, Pd, f32(decay[lo:hi]), f32(dt[lo:hi]), state,
                        _t([0, hi - lo], torch.int32), _t([0], torch.int32), o)
    got = _np(o.sum(0)[-1])
    np.testing.assert_allclose(got, want[-1], atol=2e-4)
    marked = 64.0 * x[far].reshape(H, Pd)
    assert np.abs(got[0] - marked[0]).max() < 0.1 < np.abs(marked[0]).max()          # kept
    assert np.abs(got[1]).max() < 0.01                                               # never seen again
    assert np.abs(got[2]).max() < 0.5 * np.abs(marked[2]).max()                      # faded: 0.99^497


# ----------------------------------------------------------------------------- the engine
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_layers_and_whole_prompt(name, dtype):
    from transformer_amd import Entry
    model, toks = U.engine(name, dtype), U.tokens(name, 140, 1)
    dumps = {}
    model.dump = lambda n, t: dumps.__setitem__(n, t.detach().float().cpu().numpy().copy())
    try:
        cache = model.new_cache(256)
        got = model.step(cache, [Entry(cache.alloc_slot(), toks, list(range(len(toks))))]).cpu().numpy()
    finally:
        model.dump = None
    routes = None if dtype == "float32" else \
        {int(n.split(".")[1]): t.astype(np.int64) for n, t in dumps.items() if n.endswith(".experts")}
    want, layers = U.plain(name, dtype).forward(toks, forced=routes, slack=U.SLACK)
    tol = 1e-4 if dtype == "float32" else 0.15
    for i, l in enumerate(layers):
        assert np.abs(dumps[f"run.{i}"] - l).max() < tol * max(1.0, np.abs(l).max()), f"layer {i}"
    assert U.row_error(got, want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,edit", [("A", None), ("B", None), ("D", None), ("A", "sharp"), ("D", "sharp")])
def test_cuts_agree_with_plain(name, edit, dtype):
    """Whole, portions down to two tokens, and every token alone: all against the plain model."""
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 150, 2)
    cache = model.new_cache(512, max_slots=3)
    for cuts in ([150], [2, 2, 61, 3, 64, 17], [130], []):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)                      # the next cut takes the same slot and pages
        U.check_against_plain(name, dtype, edit, toks, got, routes, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_prompt_in_portions_over_pages_and_windows(dtype):
    """400 tokens with a peaked softmax (any key inside a window may be the one a query asks for):
    portions end at and around the borders of pages, of the windows and of the recurrence's chunks;
    pages that leave every window are given back meanwhile."""
    name, edit = "A", "sharp"
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 400, 7)
    cache = model.new_cache(512, max_slots=1)
    for cuts in ([400], [257, 63, 65, 15], [64, 256, 33, 31, 16], [255, 129, 8, 7, 1], [37, 50, 3, 90, 20, 70]):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)
        U.check_against_plain(name, dtype, edit, toks, got, routes, f"cuts {cuts}")
    cache.pool.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batch_then_decoding_in_used_slots(dtype):
    from transformer_amd import Entry
    name = "A"
    model = U.engine(name, dtype)
    cache = model.new_cache(1024, max_slots=4)
    old = [cache.alloc_slot() for _ in range(4)]          # a first batch dirties every slot and page, then leaves
    model.step(cache, [Entry(s, U.tokens(name, 100 + 7 * s, 50 + s), [0]) for s in old])
    for s in old:
        cache.free_slot(s)
    lens = [1, 70, 131, 2]
    seqs = [U.tokens(name, n + 40, 10 + i) for i, n in enumerate(lens)]
    slots = [cache.alloc_slot() for _ in seqs]
    got, rows = [[] for _ in seqs], [[] for _ in seqs]
    graphs = dtype == "float32"                    # float32: recorded steps, the plain model's own routing
    rec = U.Routes(model)
    if not graphs:
        rec.__enter__()
    try:
        lg = model.step(cache, [Entry(sl, s[:n], list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu().numpy()
        at = 0
        for i, n in enumerate(lens):
            got[i].append(lg[at:at + n].copy())
            rows[i].append(slice(at, at + n))
            at += n
        live = list(range(len(seqs)))
        for step in range(40):
            if step == 25:                             # one sequence leaves early, its slot is taken again
                cache.free_slot(slots[1])
                live.remove(1)
                slots[1] = cache.alloc_slot()
            rec.next_step()
            lg = model.step(cache, [Entry(slots[i], [seqs[i][lens[i] + step]], [0]) for i in live]).cpu().numpy()
            for i in range(len(seqs)):
                rows[i].append(slice(live.index(i), live.index(i) + 1) if i in live else None)
            for j, i in enumerate(live):
                got[i].append(lg[j:j + 1].copy())
    finally:
        if not graphs:
            rec.__exit__()
    for i in range(len(seqs)):
        U.check_against_plain(name, dtype, None, seqs[i], np.concatenate(got[i]),
                              None if graphs else rec.of_rows(rows[i]), f"sequence {i}")
    cache.pool.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_match_eager_steps(dtype):
    from transformer_amd import Entry
    name = "B"
    model = U.engine(name, dtype)
    seqs = [U.tokens(name, 60, 20 + i) for i in range(3)]
    outs = []
    for graphs in (True, False):
        model.use_graphs = graphs
        try:
            cache = model.new_cache(512, max_slots=4)
            slots = [cache.alloc_slot() for _ in seqs]
            rows = []
            for t in range(60):
                lg = model.step(cache, [Entry(sl, [s[t]], [0]) for sl, s in zip(slots, seqs)])
                rows.append(lg.cpu().numpy().copy())
            outs.append(np.stack(rows))
        finally:
            model.use_graphs = True
    assert np.abs(outs[0] - outs[1]).max() < (1e-5 if dtype == "float32" else 3e-2) * np.abs(outs[1]).max()
    if dtype == "float32":          # bfloat16 against the plain model: the tests that follow the engine's routing
        want = np.stack([U.plain_logits(name, dtype, None, tuple(s)) for s in seqs], 1)
        assert U.row_error(outs[0], want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_wide_model_in_three_cuts(dtype):
    """Width 1024: heads of 128 and of 64, the experts' products on the matrix cores, products of 17
    to 64 rows that leave planes, prompts through the library and single tokens through the few-rows
    products; 330 tokens pass the borders of pages and of all three windows, and the reader's window
    is wider than its lender's."""
    name = "C"
    model, toks = U.engine(name, dtype), U.tokens(name, 330, 3)
    cache = model.new_cache(512, max_slots=2)
    for cuts in ([330], [100, 40, 70, 20, 9], [310]):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)
        U.check_against_plain(name, dtype, None, toks, got, routes, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_over_page_and_window_borders(dtype):
    name, edit = "A", "sharp"
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 330, 4)
    cache = model.new_cache(512, max_slots=1)
    slot = cache.alloc_slot()
    got, routes = U.run_cuts(model, cache, slot, toks, [30], routes=True)   # 300 single tokens over 4 borders
    U.check_against_plain(name, dtype, edit, toks, got, routes)
    if dtype == "float32":                            # once more as generation runs it: recorded steps
        cache.free_slot(slot)
        got = U.run_cuts(model, cache, cache.alloc_slot(), toks, [30])
        U.check_against_plain(name, dtype, edit, toks, got)


def test_greedy_generation_through_the_entry_point():
    import transformer_amd as ta
    from transformer_amd.engine.generate import generate
    name, dtype = "A", "float32"
    model, plain = U.engine(name, dtype), U.plain(name, dtype)
    prompts = [U.tokens(name, n, 30 + n) for n in (5, 1, 23)]
    res = generate(model, prompts, max_new_tokens=12, sample_args=ta.SampleArgs(), stop_ids=())
    for p, out in zip(prompts, res.tokens):
        assert len(out) == 12
        seq = list(p)
        for t in out:                         # the engine's choice is the plain model's best, or ties with it
            lg = plain.forward(seq)[0][-1]
            assert lg.max() - lg[t] < 1e-3
            seq.append(t)
    again = generate(model, prompts, max_new_tokens=12, sample_args=ta.SampleArgs(), stop_ids=())
    assert again.tokens == res.tokens


def test_replayer_and_command_line():
    name, dtype = "D", "float32"
    folder = U.folder(name, dtype)
    toks = U.tokens(name, 40, 5)
    want = U.plain_logits(name, dtype, None, tuple(toks))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    import tempfile
    with tempfile.TemporaryDirectory() as out:
        lines = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:30], "want": [0, 29]},
                                         {"id": "b", "tokens": toks[:1], "want": [0]}], "end": ["b"]}]
        lines += [{"step": 1 + i, "entries": [{"id": "a", "tokens": [toks[30 + i]], "want": [0]}],
                   "end": ["a"] if i == 9 else []} for i in range(10)]
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype",
                            dtype, "--out", out, "--max-tokens", "128"],
                           input="\n".join(json.dumps(l) for l in lines) + "\n", capture_output=True, text=True,
                           timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(11)]
        first = np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(3, -1)
        assert U.row_error(first, want[[0, 29, 0]]).max() < U.TOL[dtype]
        last = np.fromfile(os.path.join(out, "10.f32"), dtype="<f4").reshape(1, -1)
        assert U.row_error(last, want[39:40]).max() < U.TOL[dtype]
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--model", folder, "--dtype", dtype,
                        "--prompt", ",".join(map(str, toks[:6])), "--max-steps", "5"],
                       capture_output=True, text=True, timeout=600, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]


def test_random_weights_and_save_round_trip():
    import tempfile
    import transformer_amd as ta
    from transformer_amd import Entry
    model = ta.random_model(U.CFG_A, seed=3, dtype="float32", architecture="Saredra")
    toks = U.tokens("A", 60, 6)
    cache = model.new_cache(128)
    a = model.step(cache, [Entry(cache.alloc_slot(), toks, [59])]).cpu().numpy().copy()
    with tempfile.TemporaryDirectory() as d:
        ta.save_model(model, d)
        want = P.PlainSaredra(d).forward(toks)[0][-1:]
        again = ta.load_model(d, "float32")
        cache = again.new_cache(128)
        b = again.step(cache, [Entry(cache.alloc_slot(), toks, [59])]).cpu().numpy()
    assert np.abs(a - b).max() < 1e-6 * max(1.0, np.abs(a).max())
    assert U.row_error(a, want).max() < U.TOL["float32"]


def _draw_config(case):
    """A random Saredra configuration: any order of the two layer types, every option of each
    present or absent, sizes that are odd, equal to one another, or 1; readers of earlier layers'
    keys and values with windows of their own."""
    r = np.random.default_rng(case)
    width = int(r.choice([40, 66, 100, 136, 33, 257]))
    pick = lambda *a: a[int(r.integers(0, len(a)))]

    def rot(dim):
        if r.integers(0, 4) == 0:
            return None
        dims = dim - dim % 2 if r.integers(0, 2) else 2 * int(r.integers(1, dim // 2 + 1))
        sc = (float(pick(2.0, 8.0)), int(pick(16, 64, 512)), float(pick(4.0, 32.0)), float(pick(0.5, 1.0, 2.0))) \
            if r.integers(0, 2) else None
        return U._rot(dims, float(pick(50.0, 1e4, 1e6)), sc)

    def heads(left):
        G = int(pick(1, 2, 3))
        dk = int(pick(4, 10, 16, 24, 32))
        return U._heads(G * int(pick(1, 2, 4)), G, dk, int(pick(dk, 6, 20, 40)), float(pick(0.1, 0.25, dk ** -0.5)),
                        pick(None, 1, 5, 63, 64, 65, 100), pick(None, 2.0, 30.0), rot(dk),
                        conv=pick(None, 1, 2, 4) if left else None)

    def mlp():
        k = int(r.integers(0, 4))
        if k == 0:
            return None
        if k == 1:
            return U._dense(int(pick(8, 20, 33)))
        gc = int(pick(1, 2, 3))
        E = gc * int(pick(1, 2, 3))
        gk = int(r.integers(1, gc + 1))
        return U._moe(E, int(r.integers(1, gk * (E // gc) + 1)), int(pick(8, 20, 33)), None if gc == 1 and r.integers(0, 2) else (gc, gk))
    layers, owners = [], []
    for i in range(int(r.integers(1, 7))):
        if r.integers(0, 3) == 0:
            H = int(pick(1, 2, 3, 6))
            G = int(pick(*[g for g in (1, 2, 3, 6) if H % g == 0]))
            Pd = int(pick(2, 8, 12, 33))
            ng = int(pick(*[g for g in (1, 2, 3, H) if (H * Pd) % g == 0]))
            layers.append(U._par(heads(True), U._ssm(H, Pd, int(pick(3, 16, 40)), G, int(pick(1, 2, 4)), ng),
                                 (float(pick(1.0, 1.3)), float(pick(0.7, 1.0))), mlp()))
        elif owners and r.integers(0, 2):
            j = int(pick(*owners))
            m = dict(layers[j]["mixer"])
            m["kv_from"] = j
            m["scale"] = float(pick(0.1, 0.3))
            m.pop("mask", None)
            w = pick(None, 2, 64, 90)
            if w is not None:
                m["mask"] = {"size": w}
            layers.append(U._att(m, mlp()))
        else:
            owners.append(i)
            layers.append(U._att(heads(False), mlp()))
    cfg = {"architecture": "Saredra", "vocab": int(pick(5, 97, 300, 1001)), "width": width,
           "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    lens = [int(x) for x in r.integers(1, 150, size=int(r.integers(1, 5)))]
    return cfg, lens, r


@pytest.mark.parametrize("first", [5000, 5006, 5012, 7020])
def test_random_configurations_against_the_plain_model(first):
    """float32, the plain model's own routing, every row: a batch of unequal prompts in one step into
    poisoned pages, then eight single tokens each (recorded steps); then the same in bfloat16."""
    import tempfile
    import transformer_amd as ta
    from gpu_util import poison
    for case in range(first, first + 6):
        cfg, lens, r = _draw_config(case)
        with tempfile.TemporaryDirectory(prefix="sa_rand_") as d:
            P.make_model_folder(d, cfg, case, storage="F32")
            ref = P.PlainSaredra(d)
            model = ta.load_model(d, "float32", "cuda:0")
        toks = [[int(t) for t in r.integers(0, cfg["vocab"], size=n + 8)] for n in lens]
        cache = model.new_cache(64 * sum(-(-(n + 8) // 64) for n in lens), max_slots=len(lens))
        poison(cache)
        slots = [cache.alloc_slot() for _ in lens]
        want = [ref.forward(t)[0] for t in toks]
        what = f"case {case} {json.dumps(cfg)} prompts {lens}"
        got = model.step(cache, [ta.Entry(s, t[:n], [n - 1]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
        for i, n in enumerate(lens):
            assert U.row_error(got[i], want[i][n - 1]) < U.TOL["float32"], what
        for j in range(8):
            got = model.step(cache, [ta.Entry(s, [t[n + j]], [0]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
            for i, n in enumerate(lens):
                assert U.row_error(got[i], want[i][n + j]) < U.TOL["float32"], (what, j)
        for s in slots:
            cache.free_slot(s)
        cache.pool.check()
        with tempfile.TemporaryDirectory(prefix="sa_rand_") as d:
            P.make_model_folder(d, cfg, case, storage="BF16")
            model = ta.load_model(d, "bfloat16", "cuda:0")
        cache = model.new_cache(64 * sum(-(-(n + 8) // 64) for n in lens), max_slots=len(lens))
        poison(cache)
        slots = [cache.alloc_slot() for _ in lens]
        errs = []
        got = model.step(cache, [ta.Entry(s, t[:n], list(range(n))) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
        at = 0
        for i, n in enumerate(lens):
            errs += list(U.row_error(got[at:at + n], want[i][:n]))
            at += n
        for j in range(8):
            got = model.step(cache, [ta.Entry(s, [t[n + j]], [0]) for s, t, n in zip(slots, toks, lens)]).cpu().numpy()
            errs += [U.row_error(got[i], want[i][n + j]) for i, n in enumerate(lens)]
        errs = np.asarray(errs)
        assert np.isfinite(errs).all() and np.median(errs) < U.TOL["bfloat16"], (what, np.median(errs))
