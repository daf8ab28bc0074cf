"""Plain, slow Saredra decoder: the oracle of the Saredra tests.

Whole sequences, no cache, NumPy float64, one function per mechanism. It shares no code
with ``transformer_amd``: it reads config.json and the safetensors file itself (through the
test-suite's own reader) and states every formula once more.

Notation: T tokens, d the model's width, x the residual stream [T, d]. A weight ``W`` is
stored [out, in] and used as ``h @ W.T``.

A layer is ``x <- x + mixer(n1(x))``, then ``x <- x + ff(n2(x))`` where it has a feed-forward.
Mixers: "attention" (windowed softmax attention with capped scores, a unit added to the
softmax denominator and a sigmoid gate on the heads, which may read another layer's keys and
values) and "parallel" (a softmax branch behind short convolutions with a learned extra
denominator term per head, beside a selective state-space branch, summed with fixed weights).
The feed-forward is dense or routed among experts in groups.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from plain_llama import read_safetensors, round_bf16  # noqa: F401  (the suite's own file code)
from plain_vametar import write_safetensors  # noqa: F401

MAGNITUDE_SLOPE = 0.1       # scaled rotations multiply cos and sin by MAGNITUDE_SLOPE * ln(factor) + 1
RAMP_FLOOR = 0.001          # least width of the ramp between kept and slowed frequencies


# --------------------------------------------------------------------------
# small functions
# --------------------------------------------------------------------------
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    z = np.asarray(z, dtype=np.float64)
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def unit_rms(x, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def rotation_frequencies(rot):
    """(f [dims/2], magnitude). f_i = base^(-2i/dims). With ``scaling`` = (factor, original, fast,
    slow): the pair index at which ``t`` turns fit into ``original`` positions is n(t) = dims *
    ln(original / (2 pi t)) / (2 ln base); lo = max(floor(n(fast)), 0), hi = min(ceil(n(slow)),
    dims - 1); r_i = clamp((i - lo) / max(hi - lo, RAMP_FLOOR), 0, 1); f_i <- f_i / factor * r_i +
    f_i * (1 - r_i); cos and sin are multiplied by MAGNITUDE_SLOPE * ln(factor) + 1."""
    dims = int(rot["dims"])
    base = float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def n(t):
        return dims * np.log(original / (2.0 * np.pi * t)) / (2.0 * np.log(base))

    lo = max(np.floor(n(float(sc["fast"]))), 0.0)
    hi = min(np.ceil(n(float(sc["slow"]))), dims - 1.0)
    r = np.clip((i - lo) / max(hi - lo, RAMP_FLOOR), 0.0, 1.0)
    return f / factor * r + f * (1.0 - r), MAGNITUDE_SLOPE * np.log(factor) + 1.0


def rotate_pairs(t, positions, rot):
    """t: [T, heads, dim]. Coordinates 2i and 2i + 1, i < dims/2, of every head turn by
    position * f_i; the rest of the head passes."""
    if not rot or not rot.get("dims"):
        return t
    dims = int(rot["dims"])
    f, mag = rotation_frequencies(rot)
    a = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]          # [T, dims/2]
    c, s = (np.cos(a) * mag)[:, None, :], (np.sin(a) * mag)[:, None, :]
    out = np.array(t, dtype=np.float64, copy=True)
    u, v = t[..., 0:dims:2], t[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def causal_conv(u, w, bias=None, before=None):
    """u: [T, C], w: [C, taps]; y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros (or the rows of
    ``before``, the taps - 1 inputs in front of the first) before the start."""
    T, C = u.shape
    taps = w.shape[1]
    pad = np.zeros((taps - 1, C)) if before is None else np.asarray(before, dtype=np.float64)
    full = np.concatenate([pad, u], axis=0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += full[j:j + T] * w[:, j][None, :]
    if bias is not None:
        y = y + bias
    return y


def windowed_softmax_attention(q, k, v, scale, softcap=None, window=None, sink=None):
    """q: [T, H, dk], k: [T, G, dk], v: [T, G, dv] (all of one sequence from its first token).
    score_ij = q_i . k_j * scale, then cap * tanh(score / cap); j is seen where 0 <= i - j <
    window; p_ij = exp(s_ij) / (sum_j exp(s_ij) + exp(sink_h)), the last term only where a sink is
    given ([H] numbers; a sink of 0 adds one). Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    seen = (j <= i) if window is None else ((j <= i) & (i - j < window))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        s = np.where(seen, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[h])
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def gated_attention(h, w, p, m, positions, borrowed=None):
    """The "attention" mixer. ``borrowed``: (k after rotation, v) of the layer named by
    ``kv_from``. Returns (result [T, d], (k, v))."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rotate_pairs((h @ w[p + "q"].T).reshape(T, H, dk), positions, m.get("rot"))
    if borrowed is None:
        k = rotate_pairs((h @ w[p + "k"].T).reshape(T, G, dk), positions, m.get("rot"))
        v = (h @ w[p + "v"].T).reshape(T, G, dv)
    else:
        k, v = borrowed
    window = m["mask"]["size"] if m.get("mask") else None
    o = windowed_softmax_attention(q, k, v, m["scale"], m.get("softcap"), window, sink=np.zeros(H))
    o = o.reshape(T, H * dv) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, (k, v)


def conv_attention(h, w, p, m, positions):
    """The softmax branch of the "parallel" mixer: biased projections, a short causal convolution
    on every channel of q, k, v, scaled rotation, capped scores, a learned sink per head."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    parts = {}
    for n in "qkv":
        u = h @ w[p + n].T + w[p + n + ".b"]
        parts[n] = causal_conv(u, w[p + n + ".conv"]) if m.get("conv") else u
    q = rotate_pairs(parts["q"].reshape(T, H, dk), positions, m.get("rot"))
    k = rotate_pairs(parts["k"].reshape(T, G, dk), positions, m.get("rot"))
    v = parts["v"].reshape(T, G, dv)
    window = m["mask"]["size"] if m.get("mask") else None
    o = windowed_softmax_attention(q, k, v, m["scale"], m.get("softcap"), window, sink=w[p + "sink"])
    return o.reshape(T, H * dv) @ w[p + "o"].T


def selective_scan(x, B, C, dt, A_log, D, groups, state=None):
    """x: [T, H, P], B, C: [T, groups, N], dt: [T, H] (after softplus). Per head h with group
    g = h // (H / groups): S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T (S is [N, P]),
    y_t = S_t^T C_t + D_h x_t. Returns (y [T, H, P], last state [H, N, P])."""
    T, H, P = x.shape
    N = B.shape[2]
    S = np.zeros((H, N, P)) if state is None else np.array(state, dtype=np.float64)
    y = np.zeros((T, H, P))
    for t in range(T):
        for h in range(H):
            g = h // (H // groups)
            a = np.exp(-np.exp(A_log[h]) * dt[t, h])
            S[h] = a * S[h] + dt[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S[h].T @ C[t, g] + D[h] * x[t, h]
    return y, S


def selective_scan_sum(x, B, C, dt, A_log, D, groups):
    """The same readout as an explicit sum over earlier tokens: y_t = sum_{s <= t} (prod_{s < r <= t}
    a_r) dt_s (C_t . B_s) x_s + D x_t."""
    T, H, P = x.shape
    y = np.zeros((T, H, P))
    for h in range(H):
        g = h // (H // groups)
        la = -np.exp(A_log[h]) * dt[:, h]
        cum = np.cumsum(la)
        for t in range(T):
            wgt = np.exp(cum[t] - cum[:t + 1]) * dt[:t + 1, h] * (B[:t + 1, g] @ C[t, g])
            y[t, h] = wgt @ x[:t + 1, h] + D[h] * x[t, h]
    return y


def grouped_unit_rms(y, parts, eps):
    """y: [T, n] cut into ``parts`` equal parts, each divided by its own root mean square."""
    T, n = y.shape
    return unit_rms(y.reshape(T, parts, n // parts), eps).reshape(T, n)


def state_space(h, w, p, m, eps):
    """The state-space branch of the "parallel" mixer."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    y, _ = selective_scan(x, B, C, dt, w[p + "A_log"], w[p + "D"], G)
    y = y.reshape(T, inner) * silu(z)
    y = grouped_unit_rms(y, m["norm_groups"], eps) * w[p + "norm"]
    return y @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    return m.get("left_scale", 1.0) * conv_attention(h, w, p + "left.", m["left"], positions) + \
        m.get("right_scale", 1.0) * state_space(h, w, p + "right.", m["right"], eps)


def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def router_scores(h, w, p):
    z = h @ w[p + "router"].T
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def route(s, top, group_count=1, group_keep=1):
    """s: [E] scores. The experts form ``group_count`` equal groups of neighbours; a group counts
    as its largest score; only experts of the ``group_keep`` best groups can be chosen; among them
    the ``top`` largest (the lower index among equals). Returns the chosen experts, best first."""
    E = s.shape[0]
    allowed = np.ones(E, dtype=bool)
    if group_count > 1:
        size = E // group_count
        best = s.reshape(group_count, size).max(axis=1)
        kept = np.argsort(-best, kind="stable")[:group_keep]
        allowed[:] = False
        for g in kept:
            allowed[g * size:(g + 1) * size] = True
    masked = np.where(allowed, s, -np.inf)
    return np.argsort(-masked, kind="stable")[:top]


def close_call(s, forced, top, group_count=1, group_keep=1, slack=0.0):
    """Whether ``forced`` is what routing could choose from scores moved by at most ``slack``: its
    groups reach the weakest kept group's score within the slack, and among the experts of the
    groups then allowed each of its experts reaches the weakest chosen score within the slack."""
    E = s.shape[0]
    size = E // group_count
    mine = sorted({int(e) // size for e in forced})
    if len(set(int(e) for e in forced)) != top or len(mine) > group_keep:
        return False
    best = s.reshape(group_count, size).max(axis=1)
    if np.any(best[mine] < np.sort(best)[::-1][group_keep - 1] - slack):
        return False
    others = [int(g) for g in np.argsort(-best, kind="stable") if int(g) not in mine]
    allowed = np.concatenate([np.arange(g * size, (g + 1) * size) for g in mine + others[:group_keep - len(mine)]])
    return bool(np.all(s[np.asarray(forced, dtype=np.int64)] >= np.sort(s[allowed])[::-1][top - 1] - slack))


def moe(h, w, p, m, forced=None, slack=0.0):
    """Routed feed-forward: the chosen experts' results weighted by their scores (softmax over all
    experts, not renormalised). ``forced`` [T, top]: experts to use instead of the own choice,
    accepted only where they differ from it by a close call (``close_call`` with ``slack``).
    Returns (result, chosen [T, top])."""
    r = m["router"]
    E, top = r["experts"], r["top"]
    gc = (r.get("groups") or {}).get("count", 1)
    gk = (r.get("groups") or {}).get("keep", 1)
    s = router_scores(h, w, p)
    T, d = h.shape
    out = np.zeros((T, d))
    chosen = np.zeros((T, top), dtype=np.int64)
    for t in range(T):
        mine = route(s[t], top, gc, gk)
        if forced is not None and set(int(e) for e in forced[t]) != set(int(e) for e in mine):
            if not close_call(s[t], forced[t], top, gc, gk, slack):
                raise AssertionError(f"token {t}: experts {list(forced[t])} are no close call against "
                                     f"{list(mine)} (scores {s[t]})")
            mine = np.asarray(forced[t], dtype=np.int64)
        chosen[t] = mine
        for e in mine:
            q = f"{p}e{int(e)}."
            out[t] += s[t, e] * ((silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)) @ w[q + "down"].T)
    return out, chosen


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainSaredra:
    def __init__(self, folder):
        folder = Path(folder)
        self.c = json.loads((folder / "config.json").read_text())
        self.w = {n: np.asarray(t, dtype=np.float64) for n, t in read_safetensors(folder / "model.safetensors").items()}
        self.eps = float(self.c["norm"]["eps"])

    def forward(self, tokens, forced=None, slack=0.0, keep=None):
        """tokens: one sequence from its first token. Returns (logits [T, vocab], residual stream
        after every layer [L, T, d]). ``forced``: {layer: chosen experts [T, top]}; ``keep``: a
        dict that receives every layer's chosen experts."""
        c, w, eps = self.c, self.w, self.eps
        tokens = np.asarray(tokens, dtype=np.int64)
        T = len(tokens)
        positions = np.arange(T)
        x = w["embed"][tokens]
        stream, kv = [], {}
        for i, layer in enumerate(c["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = rms_norm(x, w[p + "norm1"], eps)
            if layer["type"] == "attention":
                src = m.get("kv_from")
                delta, kv[i] = gated_attention(h, w, p + "mix.", m, positions, None if src is None else kv[src])
            elif layer["type"] == "parallel":
                delta = parallel_mixer(h, w, p + "mix.", m, eps, positions)
            else:
                raise ValueError(f"unknown layer type {layer['type']!r}")
            x = x + delta
            mlp = layer.get("mlp")
            if mlp:
                h = rms_norm(x, w[p + "norm2"], eps)
                if mlp["kind"] == "dense":
                    x = x + dense_ff(h, w, p + "mlp.")
                else:
                    delta, chosen = moe(h, w, p + "mlp.", mlp, None if forced is None else forced.get(i), slack)
                    if keep is not None:
                        keep[i] = chosen
                    x = x + delta
            stream.append(x.copy())
        logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
        return logits, np.stack(stream)


# --------------------------------------------------------------------------
# random models for the tests
# --------------------------------------------------------------------------
def tensor_shapes(c):
    """{name: shape} of every tensor of a configuration's file."""
    d = c["width"]
    out = {"embed": (c["vocab"], d), "final.norm": (d,), "head": (c["vocab"], d)}
    for i, layer in enumerate(c["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (d,)
        if layer["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = (H * dk, d)
            if m.get("kv_from") is None:
                out[p + "mix.k"], out[p + "mix.v"] = (G * dk, d), (G * dv, d)
            out[p + "mix.g"], out[p + "mix.o"] = (H * dv, d), (d, H * dv)
        else:
            a, b = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            for n, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                out[q + n], out[q + n + ".b"] = (rows, d), (rows,)
                if a.get("conv"):
                    out[q + n + ".conv"] = (rows, a["conv"])
            out[q + "sink"], out[q + "o"] = (H,), (d, H * dv)
            q = p + "mix.right."
            inner, gn = b["heads"] * b["vdim"], b["groups"] * b["state"]
            out[q + "in"] = (2 * inner + 2 * gn + b["heads"], d)
            out[q + "conv"], out[q + "conv.b"] = (inner + 2 * gn, b["conv"]), (inner + 2 * gn,)
            for n in ("dt_bias", "A_log", "D"):
                out[q + n] = (b["heads"],)
            out[q + "norm"], out[q + "o"] = (inner,), (d, inner)
        mlp = layer.get("mlp")
        if mlp:
            out[p + "norm2"] = (d,)
            if mlp["kind"] == "dense":
                ff = mlp["ff"]
                out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = (ff, d), (ff, d), (d, ff)
            else:
                ff = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    q = f"{p}mlp.e{e}."
                    out[q + "gate"], out[q + "up"], out[q + "down"] = (ff, d), (ff, d), (d, ff)
                out[p + "mlp.router"] = (mlp["router"]["experts"], d)
    return out


def random_weights(c, seed, edit=None):
    """bfloat16-representable float32 weights: matrices N(0, 1/sqrt(in)), norm weights around one,
    biases, sinks and the state-space constants small; the router's rows larger, so that choices are
    seldom close. ``edit(weights)`` may change them before they are rounded."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(c).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm") and len(shape) == 1:
            t = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "conv":
            t = rng.standard_normal(shape) * 0.5
        elif leaf == "b":
            t = rng.standard_normal(shape) * 0.2
        elif leaf == "sink":
            t = rng.standard_normal(shape) * 1.0
        elif leaf == "dt_bias":
            t = rng.uniform(-3.0, 0.5, shape)
        elif leaf == "A_log":
            t = rng.uniform(-1.5, 1.0, shape)
        elif leaf == "D":
            t = rng.standard_normal(shape)
        elif leaf == "router":
            t = rng.standard_normal(shape) * (3.0 / np.sqrt(shape[1]))
        elif leaf == "embed":
            t = rng.standard_normal(shape)
        else:
            t = rng.standard_normal(shape) / np.sqrt(shape[-1])
        w[name] = t
    if edit is not None:
        edit(w)
    return {n: round_bf16(np.asarray(t, dtype=np.float32)) for n, t in w.items()}


def make_model_folder(folder, c, seed, storage="BF16", edit=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(c))
    write_safetensors(folder / "model.safetensors", random_weights(c, seed, edit), storage)
    return folder
