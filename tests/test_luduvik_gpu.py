"""The Luduvik decoder on the GPU against the plain implementation in ``plain_luduvik``.

Each mechanism alone (its kernels against the plain function, with cache and state carried over
cuts), then the engine: layers, whole prompts, portions, token-by-token decoding, unequal
batches, slots and pages used again, recorded steps, far keys and keys at the borders of pages,
long decoding, greedy generation, the replayer and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import luduvik_util as U
import plain_luduvik as P

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
@pytest.mark.parametrize("d", [72, 90, 1024, 4100])
@pytest.mark.parametrize("n", [1, 2, 3])
def test_mean_of_normed_branches(d, n):
    from transformer_amd import kernels
    rng = np.random.default_rng(d + n)
    nt = 7
    # the first branch arrives as three planes that add up, the others as one; very unequal sizes,
    # which the norms level before the mean
    deltas = [10.0 ** i * rng.standard_normal((3, nt, d) if i == 0 else (nt, d)) for i in range(n)]
    ws = [1 + 0.2 * rng.standard_normal(d) for _ in range(n)]
    out = torch.full((nt, d), float("nan"), device=DEV)
    kernels.normed_mean([_t(a) for a in deltas], [_t(w) for w in ws], 1e-5, out)
    f32 = [a.astype(np.float32).astype(np.float64) for a in deltas]
    want = sum(P.rms_norm(a.sum(0) if a.ndim == 3 else a, w, 1e-5) for a, w in zip(f32, ws)) / n
    assert np.abs(_np(out) - want).max() < 2e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("limit", [0.5, 1.0, 7.0])
def test_limited_gate(dtype, limit):
    from transformer_amd import kernels
    rng = np.random.default_rng(3)
    n = 37
    rows = _bf(2.5 * rng.standard_normal((9, 2 * n + 5)), dtype)            # rows wider than [gate | up]
    rows[0, :4] = [limit, -limit, 3 * limit, -3 * limit]                   # the gate: at and beyond the limit
    rows[1, :2], rows[1, n:n + 2] = [0.3, 0.3], [-3 * limit, -limit]
    rows[0, n:n + 4] = [limit, -limit, 3 * limit, 0.5 * limit]             # the up branch: limited on both sides
    g, u = np.minimum(rows[:, :n], limit), np.clip(rows[:, n:2 * n], -limit, limit)
    want = g * P.sigmoid(P.GATE_SLOPE * g) * (u + 1.0)
    out = torch.empty(9, n, dtype=TD[dtype], device=DEV)
    kernels.glu_limit(_t(rows, TD[dtype])[:, :2 * n], out, limit)
    _close(_np(out), want, dtype)
    # the gate has an upper limit only; the up branch is limited on both sides
    assert float(out[0, 2]) == float(out[0, 0]) and (limit > 1 or abs(float(out[0, 3])) > abs(float(out[0, 1])) * 1.05)
    assert float(out[1, 0]) == float(out[1, 1])
    kernels.glu_limit(_t(rows, TD[dtype])[:, :2 * n], out, limit, 1.0, 0.0)                  # other constants
    _close(_np(out), g * P.sigmoid(g) * u, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(3072, 4096, 0), (24, 40, 8), (24, 40, 4), (20, 36, 0), (6144, 8192, 2048)])
def test_silu_in_place_on_the_first_columns_of_wider_rows(dtype, geom):
    """q, k, v of the lightning mixer are activated in place inside the rows [q | k | v | gate];
    rows that start on 16 bytes take the kernel with wide loads, the others the plain one."""
    from transformer_amd import kernels
    n, width, first = geom
    rng = np.random.default_rng(n)
    rows = _bf(3 * rng.standard_normal((5, width)), dtype)
    t = _t(rows, TD[dtype])
    kernels.activation(t[:, first:first + n], t[:, first:first + n], "silu")
    want = rows.copy()
    want[:, first:first + n] = P.silu(rows[:, first:first + n])
    _close(_np(t), want, dtype)
    assert np.array_equal(_np(t)[:, first + n:], rows[:, first + n:]) and np.array_equal(_np(t)[:, :first], rows[:, :first])


@pytest.mark.parametrize("geom", [(5, 2), (3, 3), (1, 1), (16, 1), (9, 4), (64, 6)])
def test_router_bias_and_softmax_over_the_chosen(geom):
    from transformer_amd import kernels
    E, top = geom
    rng = np.random.default_rng(E * 10 + top)
    nt = 50
    z = rng.standard_normal((nt, E + 3)).astype(np.float32)                # more columns than experts
    b = (2.0 * rng.standard_normal(E)).astype(np.float32)                  # a bias that changes who is chosen
    chosen = torch.empty(nt, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(nt, top, device=DEV)
    kernels.moe_route(_t(z), E, top, chosen, weight, "softmax", True, bias=_t(b))
    want_c, want_w = P.route(z[:, :E].astype(np.float64) + b, top)
    got_c, got_w = chosen.cpu().numpy(), _np(weight)
    for t in range(nt):
        order = np.argsort(got_c[t])
        assert sorted(got_c[t]) == sorted(want_c[t]), t
        np.testing.assert_allclose(got_w[t][order], want_w[t][np.argsort(want_c[t])], atol=1e-6)
    np.testing.assert_allclose(got_w.sum(1), 1.0, atol=1e-6)
    if E > 1:
        plain_c, _ = P.route(z[:, :E].astype(np.float64), top)
        assert any(sorted(a) != sorted(c) for a, c in zip(plain_c, want_c)) or top == E


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(5, 2, 24, 72, 40, 1.0, 0.7), (3, 3, 16, 72, None, 2.0, 0.0), (1, 1, 32, 64, 8, 1.0, 1.0),
                                  (7, 1, 20, 90, 12, 0.5, 3.0), (12, 3, 48, 328, 96, 1.25, 0.9), (8, 2, 256, 1024, 512, 1.5, 1.0)])
def test_routed_limited_experts_part(dtype, geom):
    """The routed feed-forward as the block runs it (routing with the bias, ordering, both products,
    the limited gate, the shared expert, the other sublayer's delta taken into the sum) against the
    plain function."""
    from transformer_amd.config.spec import RoutedMLPSpec
    from transformer_amd.parts.linear import Workspace
    from transformer_amd.parts.base import build_part
    E, top, ff, d, sff, limit, slimit = geom
    rng = np.random.default_rng(E + top + ff)
    m = {"router": {"experts": E, "top": top}, "expert": {"ff": ff, "limit": limit}}
    shapes = {"router": (E, d), "router.b": (E,)}
    for e in range(E):
        shapes.update({f"e{e}.gate": (ff, d), f"e{e}.up": (ff, d), f"e{e}.down": (d, ff)})
    if sff is not None:
        m["shared"] = {"ff": sff, "limit": slimit}
        shapes.update({"shared.gate": (sff, d), "shared.up": (sff, d), "shared.down": (d, sff)})
    w = {n: _bf((4.0 if n.startswith("router") else 2.0) * rng.standard_normal(s) / np.sqrt(s[-1] if len(s) > 1 else 1.0), dtype)
         for n, s in shapes.items()}
    spec = RoutedMLPSpec(hidden=d, experts=E, top=top, intermediate=ff, score="softmax", renormalize=True,
                         weight_on="output", shared_intermediate=sff, shared_gate=False, router_bias=True,
                         form="limited_glu", limit=limit, shared_limit=slimit, gate_slope=1.702, up_shift=1.0)
    part = build_part(spec, TD[dtype], DEV)
    mat = lambda a: _t(a, TD[dtype])
    tensors = {"router.weight": mat(w["router"]), "router.bias": _t(w["router.b"]),
               "experts.gate_up.weight": mat(np.concatenate([w[f"e{e}.{n}"] for e in range(E) for n in ("gate", "up")])),
               "experts.down.weight": mat(np.concatenate([w[f"e{e}.down"] for e in range(E)]))}
    if sff is not None:
        tensors["shared.gate_up.weight"] = mat(np.concatenate([w["shared.gate"], w["shared.up"]]))
        tensors["shared.down.weight"] = mat(w["shared.down"])
    part.bind(tensors)

    class Ctx:
        ws, dump = Workspace(DEV), None
    for nt in (1, 9, 150):
        h = _bf(rng.standard_normal((nt, d)), dtype)
        extra = rng.standard_normal((2, nt, d)).astype(np.float32)
        chosen = {}
        Ctx.dump = lambda name, t: chosen.__setitem__(name, t.cpu().numpy().astype(np.int64))
        delta, bias = part.run(mat(h), Ctx, extra=_t(extra))
        assert bias is None
        want = P.moe(h, w, "", m, forced=None if dtype == "float32" else chosen["experts"], slack=0.05)
        _close(_np(delta), want + extra.astype(np.float64).sum(0), dtype, f"{nt} rows")


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
@pytest.mark.parametrize("geom", [(6, 2, 20, 12, 8, (8.0, 1.0, 4.0, 64)), (4, 4, 16, 24, 0, None), (1, 1, 16, 16, 16, None),
                                  (5, 5, 7, 11, 6, None), (2, 1, 34, 6, 34, (3.0, 1.0, 3.0, 32)), (4, 1, 8, 40, 2, None),
                                  (8, 2, 128, 64, 64, (4.0, 1.0, 4.0, 256))])
def test_softmax_branch_pieces(dtype, geom):
    """Heads normed one by one with a weight of the head's width, the first coordinates of every
    head rotated with slowed frequencies, keys and values into shuffled pages; a prompt in two
    portions, two single tokens and another portion, against the plain function."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    from transformer_amd.parts.position import scaled_frequencies
    H, G, dk, dv, rot, scaling = geom
    rng = np.random.default_rng(H * 7 + dk)
    T, eps, scale, base = 150, 1e-5, 0.21, 500.0
    rows = _bf(rng.standard_normal((T, (H + G) * dk + G * dv)), dtype)
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": scale}
    if rot:
        m["rot"] = {"dims": rot, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    sq, sk, sv = _selectors([H * dk, G * dk, G * dv])
    w = {"q": sq, "k": sk, "v": sv, "o": np.eye(H * dv), "q.norm": 1 + 0.3 * rng.standard_normal(dk),
         "k.norm": 1 + 0.3 * rng.standard_normal(dk)}
    want = P.softmax_attention(rows, w, "", m, eps, np.arange(T))
    kc = torch.full((9, G, PAGE, dk), float("nan"), dtype=TD[dtype], device=DEV)
    vc = torch.full((9, G, dv, PAGE), float("nan"), dtype=TD[dtype], device=DEV)
    pages = np.array([7, 2, 5])
    inv = _t(scaled_frequencies(rot, base, scaling)) if rot else None
    if rot:
        np.testing.assert_allclose(scaled_frequencies(rot, base, scaling), P.rotation_frequencies(m["rot"]), rtol=1e-12)
    got, at = [], 0
    for n in (70, 58, 1, 1, 20):
        p = np.arange(at, at + n)
        qkv = _t(rows[p], TD[dtype])
        angles = K.rope_table(_t(p, torch.int32), inv, torch.empty(n, rot // 2, 2, device=DEV)) if rot else None
        dest = _t(pages[p // PAGE] * PAGE + p % PAGE, torch.int32)
        K.qk_prepare(qkv, H, G, dk, dv, eps, _t(w["q.norm"]), _t(w["k.norm"]), angles, rot, dest=dest, kcache=kc,
                     vcache=vc, per_head=True)
        o = torch.empty(n, H * dv, dtype=TD[dtype], device=DEV)
        K.attention_generic_dv(qkv, o, kc, vc, _t([pages], torch.int32), _t([0, n], torch.int32), _t([at], torch.int32),
                               n, H, G, dk, dv, scale)
        got.append(_np(o))
        at += n
    _close(np.concatenate(got), want, dtype, scale=1.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("where", ["prompt", "decode"])
@pytest.mark.parametrize("mark", [0, 3, 63, 64, 127, 128, 298])
def test_one_key_stands_out(where, dtype, mark):
    """The last query points at ONE earlier key (the first token, a few back, hundreds back, the
    last and the first of a page): after the heads' norms with large gains its score stands out,
    so the result is that key's value. The energy sits in coordinates that do not rotate; the
    rotated ones carry noise."""
    from transformer_amd import kernels as K
    from transformer_amd.kernels import PAGE
    H, G, dk, dv, rot, T = 4, 2, 32, 24, 8, 300
    rng = np.random.default_rng(mark)
    q, k = 0.05 * rng.standard_normal((T, H * dk)), 0.05 * rng.standard_normal((T, G * dk))
    v = _bf(rng.standard_normal((T, G * dv)), dtype)
    k.reshape(T, G, dk)[mark, :, rot:rot + 4] = 3.0
    q.reshape(T, H, dk)[T - 1, :, rot:rot + 4] = 3.0
    rows = _bf(np.concatenate([q, k, v], 1), dtype)
    gain = _t(np.full(dk, 4.0))
    pages = np.array([4, 1, 3, 0, 5])
    kc = torch.full((6, G, PAGE, dk), float("nan"), dtype=TD[dtype], device=DEV)
    vc = torch.full((6, G, dv, PAGE), float("nan"), dtype=TD[dtype], device=DEV)
    inv = _t(100.0 ** (-2.0 * np.arange(rot // 2) / rot))
    nq = 1 if where == "decode" else 45
    for p in (np.arange(0, T - nq), np.arange(T - nq, T)):
        qkv = _t(rows[p], TD[dtype])
        angles = K.rope_table(_t(p, torch.int32), inv, torch.empty(len(p), rot // 2, 2, device=DEV))
        dest = _t(pages[p // PAGE] * PAGE + p % PAGE, torch.int32)
        K.qk_prepare(qkv, H, G, dk, dv, 1e-6, gain, gain, angles, rot, dest=dest, kcache=kc, vcache=vc, per_head=True)
    o = torch.empty(nq, H * dv, dtype=TD[dtype], device=DEV)
    K.attention_generic_dv(qkv, o, kc, vc, _t([pages], torch.int32), _t([0, nq], torch.int32), _t([T - nq], torch.int32),
                           nq, H, G, dk, dv, 0.25)
    want = np.repeat(v[mark].reshape(G, dv), H // G, axis=0).reshape(-1)
    assert np.abs(_np(o[-1]) - want).max() < (1e-3 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geom", [(3, 12, 20, 12, "retention"), (1, 64, 64, 0, "lightning"), (5, 4, 4, 0, "lightning"),
                                  (2, 33, 5, 2, "retention"), (8, 128, 128, 128, "retention"), (4, 96, 160, 32, "retention"),
                                  (16, 64, 64, 0, "lightning"), (2, 16, 8, 0, "retention")])
def test_decay_linear_attention_pieces(dtype, geom):
    """Rotation of q and k in place, the recurrence with the state carried over cuts of many, one
    and two tokens, the norm (per head without a weight, or over all heads with one) and the gate;
    three sequences of unequal lengths in slots that held something else; decays of 0 and 1."""
    from transformer_amd import kernels as K
    H, dk, dv, rot, kind = geom
    rng = np.random.default_rng(H * 100 + dk)
    lens, eps = [37, 1, 12], 1e-5
    decay = np.array(([1.0, 0.0, 0.9, 0.999, 0.5] * 4)[:H])
    if H == 1:
        decay = np.array([0.98])
    nk, nv = H * dk, H * dv
    rotd = {"dims": rot, "base": 100.0} if rot else None
    seqs = [_bf(rng.standard_normal((L + 5, 2 * nk + 2 * nv)), dtype) for L in lens]
    nw = 1 + 0.2 * rng.standard_normal(nv)

    def plain_one(rows):
        T = len(rows)
        q, k = rows[:, :nk].reshape(T, H, dk), rows[:, nk:2 * nk].reshape(T, H, dk)
        v, g = rows[:, 2 * nk:2 * nk + nv].reshape(T, H, dv), rows[:, 2 * nk + nv:]
        if kind == "lightning":
            o, _ = P.decayed_linear_attention(_bf(P.silu(q), dtype), _bf(P.silu(k), dtype), _bf(P.silu(v), dtype), decay)
            return P.rms_norm(o.reshape(T, nv), nw, eps) * P.sigmoid(g), o
        if rotd:
            q, k = P.rotate_half(q, np.arange(T), rotd), P.rotate_half(k, np.arange(T), rotd)
        o, _ = P.decayed_linear_attention(_bf(q, dtype), _bf(k, dtype) * dk ** -0.5, v, decay)
        return P.unit_rms(o, eps).reshape(T, nv) * P.silu(g), o
    state = torch.full((5, H, dk, dv), 3.0, device=DEV)
    slots = [3, 0, 4]
    for s in slots:
        state[s] = 0.0                                                      # a sequence starts from zero
    inv = _t(100.0 ** (-2.0 * np.arange(rot // 2) / rot)) if rot else None
    got = [[] for _ in lens]
    done = [0] * len(lens)
    for part in (lambda L: L, lambda L: 1, lambda L: 2, lambda L: 2):
        rows = [s[a:a + part(L)] for s, L, a in zip(seqs, lens, done)]
        proj = _t(np.concatenate(rows), TD[dtype])
        nt = proj.shape[0]
        cu = _t(np.concatenate([[0], np.cumsum([len(r) for r in rows])]), torch.int32)
        qkv = proj[:, :2 * nk + nv]
        if kind == "lightning":
            K.activation(qkv, qkv, "silu")
        elif rot:
            pos = np.concatenate([np.arange(a, a + len(r)) for a, r in zip(done, rows)])
            angles = K.rope_table(_t(pos, torch.int32), inv, torch.empty(nt, rot // 2, 2, device=DEV))
            K.qk_prepare(qkv, H, H, dk, dv, eps, None, None, angles, rot, k_inplace=True)
        o = torch.empty(K.gla_row_parts(dk), nt, H, dv, device=DEV)
        K.decay_recurrent(proj, 0, nk, 2 * nk, H, dk, dv, _t(decay), 1.0 if kind == "lightning" else dk ** -0.5,
                          state, cu, _t(slots, torch.int32), o)
        out = torch.empty(nt, nv, dtype=TD[dtype], device=DEV)
        gate = proj[:, 2 * nk + nv:]
        if kind == "lightning":
            K.head_norm_gate(o.view(o.shape[0], nt, 1, nv), gate, 1, nv, _t(nw), eps, out, "sigmoid")
        else:
            K.head_norm_gate(o, gate, H, dv, None, eps, out, "silu")
        at = 0
        for i, r in enumerate(rows):
            got[i].append((_np(out[at:at + len(r)]), _np(o.sum(0)[at:at + len(r)])))
            at += len(r)
            done[i] += len(r)
    for i, s in enumerate(seqs):
        want, want_o = plain_one(s)
        _close(np.concatenate([g[1] for g in got[i]]), want_o.reshape(want_o.shape[0], H, dv), dtype, f"readout {i}",
               scale=1.0 if dtype == "float32" else 0.5)
        _close(np.concatenate([g[0] for g in got[i]]), want, dtype, f"sequence {i}", scale=2.0)
    assert float(state[1].min()) == 3.0 and float(state[2].max()) == 3.0    # slots of others stay as they are


@pytest.mark.parametrize("where", ["prompt", "decode"])
def test_a_far_token_in_the_state(where):
    """Decay 1 keeps a token for ever: the last query points at the key of token 2 among 500, whose
    value is then what the head reads out; with decay 0 the same query reads the last token only;
    with 0.99 the far token has faded (0.99^497 < 0.01) beside what came later."""
    from transformer_amd import kernels as K
    H, dk, dv, T, far = 3, 16, 12, 500, 2
    rng = np.random.default_rng(8)
    q, k = 0.01 * rng.standard_normal((T, H, dk)), 0.01 * rng.standard_normal((T, H, dk))
    v = rng.standard_normal((T, H, dv))
    k[far, :, 5], q[T - 1, :, 5], k[T - 1, :, 5] = 8.0, 8.0, 1.0
    decay = np.array([1.0, 0.0, 0.99])
    rows = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1)
    state = torch.zeros(2, H, dk, dv, device=DEV)
    cuts = [T] if where == "prompt" else [T - 40] + [1] * 40
    at = 0
    for n in cuts:
        o = torch.empty(K.gla_row_parts(dk), n, H, dv, device=DEV)
        K.decay_recurrent(_t(rows[at:at + n]), 0, H * dk, 2 * H * dk, H, dk, dv, _t(decay), 1.0, state,
                          _t([0, n], torch.int32), _t([1], torch.int32), o)
        at += n
    last = _np(o.sum(0)[-1])
    score = np.einsum("hk,jhk->jh", q[T - 1], k)                           # the last query against every key
    want = np.einsum("jh,jhv->hv", score * decay[None, :] ** (T - 1 - np.arange(T))[:, None], v)
    np.testing.assert_allclose(last, want, atol=2e-3)
    # the far token's 64 v beside the last token's own and 500 small ones
    assert np.abs(want[0] - score[T - 1, 0] * v[T - 1, 0] - 64.0 * v[far, 0]).max() < 8.0 < np.abs(64.0 * v[far, 0]).max()
    np.testing.assert_allclose(want[1], score[T - 1, 1] * v[T - 1, 1], atol=1e-9)
    assert abs(score[far, 2]) * decay[2] ** (T - 1 - far) < 0.5            # faded: 64 times 0.99^497


# ----------------------------------------------------------------------------- the engine
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_layers_and_whole_prompt(name, dtype):
    from transformer_amd import Entry
    model, toks = U.engine(name, dtype), U.tokens(name, 90, 1)
    dumps = {}
    model.dump = lambda n, t: dumps.__setitem__(n, t.detach().float().cpu().numpy().copy())
    try:
        cache = model.new_cache(256)
        got = model.step(cache, [Entry(cache.alloc_slot(), toks, list(range(len(toks))))]).cpu().numpy()
    finally:
        model.dump = None
    layers = []
    routes = None if dtype == "float32" else \
        {int(n.split(".")[1]): t.astype(np.int64) for n, t in dumps.items() if n.endswith(".experts")}
    want = U.plain(name, dtype).forward(toks, layers, routes=routes)
    tol = 1e-4 if dtype == "float32" else 0.15
    for i, l in enumerate(layers):
        assert np.abs(dumps[f"run.{i}"] - l).max() < tol * max(1.0, np.abs(l).max()), f"layer {i}"
    assert U.row_error(got, want).max() < U.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,edit", [("A", None), ("B", None), ("D", None), ("A", "sharp"), ("B", "sharp")])
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
def test_long_prompt_in_portions_over_pages(dtype):
    """400 tokens with a peaked softmax (any key of the 400 may be the one a query asks for) and
    decays up to 1: portions end at and around the borders of pages and the recurrence's chunks."""
    name, edit = "A", "sharp"
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 400, 7)
    cache = model.new_cache(512, max_slots=1)
    for cuts in ([400], [257, 63, 65, 15], [64, 256, 33, 31, 16], [255, 129, 8, 7, 1]):
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
    """Width 1024: heads of 128 and of 64 take the matrix-core attention (values narrower than the
    keys among them), the experts' products the matrix cores, products of 17 to 64 rows leave
    planes, prompts go to the library and single tokens to the few-rows products; 260 tokens pass
    the borders of pages."""
    name = "C"
    model, toks = U.engine(name, dtype), U.tokens(name, 260, 3)
    cache = model.new_cache(512, max_slots=2)
    for cuts in ([260], [100, 40, 70, 20, 9], [250]):
        slot = cache.alloc_slot()
        got, routes = U.run_cuts(model, cache, slot, toks, cuts, routes=True)
        cache.free_slot(slot)
        U.check_against_plain(name, dtype, None, toks, got, routes, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_over_page_borders(dtype):
    name, edit = "A", "sharp"
    model, toks = U.engine(name, dtype, edit), U.tokens(name, 330, 4)
    cache = model.new_cache(512, max_slots=1)
    slot = cache.alloc_slot()
    got, routes = U.run_cuts(model, cache, slot, toks, [60], routes=True)   # 270 single tokens over 4 borders
    U.check_against_plain(name, dtype, edit, toks, got, routes)
    if dtype == "float32":                            # once more as generation runs it: recorded steps
        cache.free_slot(slot)
        got = U.run_cuts(model, cache, cache.alloc_slot(), toks, [60])
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
            lg = plain.forward(seq)[-1]
            assert lg.max() - lg[t] < 1e-3
            seq.append(t)
    again = generate(model, prompts, max_new_tokens=12, sample_args=ta.SampleArgs(), stop_ids=())
    assert again.tokens == res.tokens


def test_replayer_and_command_line():
    name, dtype = "B", "float32"
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
    model = ta.random_model(U.CFG_B, seed=3, dtype="float32", architecture="Luduvik")
    toks = U.tokens("B", 20, 6)
    cache = model.new_cache(128)
    a = model.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy().copy()
    with tempfile.TemporaryDirectory() as d:
        ta.save_model(model, d)
        want = P.PlainLuduvik(d).forward(toks)[-1:]
        again = ta.load_model(d, "float32")
        cache = again.new_cache(128)
        b = again.step(cache, [Entry(cache.alloc_slot(), toks, [19])]).cpu().numpy()
    assert np.abs(a - b).max() < 1e-6 * max(1.0, np.abs(a).max())
    assert U.row_error(a, want).max() < U.TOL["float32"]


def _draw_config(case):
    """A random Luduvik configuration: any order of the two layer types, every option of each
    present or absent, sizes that are odd, equal to one another, or 1."""
    r = np.random.default_rng(case)
    width = int(r.choice([40, 66, 100, 136, 33, 257]))
    pick = lambda *a: a[int(r.integers(0, len(a)))]

    def rot(dim, scaled):
        if r.integers(0, 4) == 0:
            return None
        dims = dim - dim % 2 if r.integers(0, 2) else 2 * int(r.integers(1, dim // 2 + 1))
        sc = (float(pick(2.0, 8.0)), 1.0, float(pick(2.0, 4.0)), int(pick(16, 64, 512))) if scaled and r.integers(0, 2) else None
        return U._rot(dims, float(pick(50.0, 1e4, 1e6)), sc) if dims else None

    def lin(with_rot):
        H, dk = int(pick(1, 2, 3, 5)), int(pick(2, 8, 12, 20, 33, 64))
        return U._lin(H, dk, int(pick(dk, 4, 10, 24)), [float(pick(0.0, 0.5, 0.9, 0.99, 0.999, 1.0)) for _ in range(H)],
                      rot(dk, False) if with_rot else None)
    layers = []
    for _ in range(int(r.integers(1, 6))):
        mlp = None
        if r.integers(0, 4):
            E = int(pick(1, 2, 5, 9, 16))
            mlp = U._moe(E, int(r.integers(1, E + 1)), int(pick(8, 20, 33)), float(pick(0.5, 1.0, 7.0)),
                         shared=None if r.integers(0, 2) else (int(pick(6, 24)), float(pick(0.5, 2.0))))
        if r.integers(0, 2):
            layers.append(U._lit(lin(False), mlp))
            continue
        G = int(pick(1, 2, 3))
        dk = int(pick(4, 10, 16, 24, 32))
        left = U._left(G * int(pick(1, 2, 4)), G, dk, int(pick(dk, 6, 20, 40)), float(pick(0.1, 0.25, dk ** -0.5)), rot(dk, True))
        layers.append(U._par(left, lin(True), mlp))
    cfg = {"architecture": "Luduvik", "vocab": int(pick(5, 97, 300, 1001)), "width": width,
           "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    lens = [int(x) for x in r.integers(1, 150, size=int(r.integers(1, 5)))]
    return cfg, lens, r


@pytest.mark.parametrize("first", [3000, 3006, 3012])
def test_random_configurations_against_the_plain_model(first):
    """float32, the plain model's own routing, every row: a batch of unequal prompts in one step into
    poisoned pages, then eight single tokens each (recorded steps); then the same in bfloat16."""
    import tempfile
    import transformer_amd as ta
    from gpu_util import poison
    for case in range(first, first + 6):
        cfg, lens, r = _draw_config(case)
        with tempfile.TemporaryDirectory(prefix="lu_rand_") as d:
            P.make_model_folder(d, cfg, case, storage="F32")
            ref = P.PlainLuduvik(d)
            model = ta.load_model(d, "float32", "cuda:0")
        toks = [[int(t) for t in r.integers(0, cfg["vocab"], size=n + 8)] for n in lens]
        cache = model.new_cache(64 * sum(-(-(n + 8) // 64) for n in lens), max_slots=len(lens))
        poison(cache)
        slots = [cache.alloc_slot() for _ in lens]
        want = [ref.forward(t) for t in toks]
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
        with tempfile.TemporaryDirectory(prefix="lu_rand_") as d:
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
