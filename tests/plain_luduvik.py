"""Plain, slow Luduvik decoder: the oracle of the Luduvik tests.

Whole sequences, no cache, NumPy float64, one function per mechanism. It shares no code
with ``transformer_amd``: it reads config.json and the safetensors file itself (through the
test-suite's own reader) and states every formula once more.

Notation: T tokens, d the model's width, x the residual stream [T, d]. A weight ``W`` is
stored [out, in] and used as ``h @ W.T``.

A layer is ``x <- x + mixer(n(x)) + ff(n(x))`` with ONE norm n in front of both sublayers.
Mixers: "lightning" (linear attention with a fixed decay per head behind silu maps) and
"parallel" (softmax attention with normed, partly rotated heads beside a retention branch,
each result normed over the model width, then averaged). The feed-forward routes every token
to its ``top`` experts by the largest router logits and adds a shared expert.
"""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from plain_llama import read_safetensors, round_bf16  # noqa: F401  (the suite's own file code)
from plain_vametar import write_safetensors  # noqa: F401

GATE_SLOPE = 1.702      # the experts' gate is g * sigmoid(GATE_SLOPE * g)


# --------------------------------------------------------------------------
# small functions
# --------------------------------------------------------------------------
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def unit_rms(x, eps):
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def rotation_frequencies(rot):
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` the long wavelengths are slowed:
    wavelength above original/low: f / factor; below original/high: f; between: a blend
    whose share of the unscaled f grows linearly in original/wavelength."""
    dims = rot["dims"]
    f = float(rot["base"]) ** (-2.0 * np.arange(dims // 2, dtype=np.float64) / dims)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = f.copy()
        for i, fi in enumerate(f):
            wl = 2.0 * np.pi / fi
            if wl > orig / low:
                out[i] = fi / factor
            elif wl >= orig / high:
                s = (orig / wl - low) / (high - low)
                out[i] = (1.0 - s) * fi / factor + s * fi
        f = out
    return f


def rotate_half(t, positions, rot):
    """t: [T, heads, dh]. Coordinate i < dims/2 of every head is paired with i + dims/2 and the
    pair turns by position * f_i; coordinates from ``dims`` on stay."""
    dims = rot["dims"]
    half = dims // 2
    out = np.array(t, dtype=np.float64)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * rotation_frequencies(rot)
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = t[..., :half], t[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def softmax_attention(h, w, p, m, eps, positions):
    """The softmax branch: grouped heads, q and k normed per head with ONE weight of the head's
    width, the first rot.dims coordinates rotated, causal softmax of q.k * scale."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, dk)
    k = (h @ w[p + "k"].T).reshape(T, G, dk)
    v = (h @ w[p + "v"].T).reshape(T, G, dv)
    q = rms_norm(q, w[p + "q.norm"], eps)
    k = rms_norm(k, w[p + "k.norm"], eps)
    if m.get("rot"):
        q, k = rotate_half(q, positions, m["rot"]), rotate_half(k, positions, m["rot"])
    out = np.zeros((T, H, dv))
    mask = np.tril(np.ones((T, T), dtype=bool))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        s = np.where(mask, s, -np.inf)
        s = s - s.max(axis=-1, keepdims=True)
        e = np.exp(s)
        out[:, hd] = (e / e.sum(axis=-1, keepdims=True)) @ v[:, g]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def decayed_linear_attention(q, k, v, decay, state=None):
    """q, k [T, H, dk], v [T, H, dv], decay [H]: S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t.
    Returns (o [T, H, dv], last S [H, dk, dv])."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((H, dk, dv)) if state is None else np.array(state, dtype=np.float64)
    o = np.zeros((T, H, dv))
    decay = np.asarray(decay, dtype=np.float64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hkv,hk->hv", S, q[t])
    return o, S


def decayed_linear_attention_sum(q, k, v, decay):
    """The same readout written as a sum over earlier tokens (no state), for cross-checks."""
    T, H, dk = q.shape
    o = np.zeros((T, H, v.shape[-1]))
    decay = np.asarray(decay, dtype=np.float64)
    for t in range(T):
        for j in range(t + 1):
            o[t] += (decay ** (t - j))[:, None] * np.einsum("hk,hk->h", q[t], k[j])[:, None] * v[j]
    return o


def retention(h, w, p, m, eps, positions):
    """The retention branch: rotated q and k, k scaled by dk^-1/2 after the rotation, the
    decayed sum, every head's readout divided by its root mean square, times silu(gate)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(T, H, dk)
    k = (h @ w[p + "k"].T).reshape(T, H, dk)
    v = (h @ w[p + "v"].T).reshape(T, H, dv)
    if m.get("rot"):
        q, k = rotate_half(q, positions, m["rot"]), rotate_half(k, positions, m["rot"])
    k = k * dk ** -0.5
    o, _ = decayed_linear_attention(q, k, v, m["decay"])
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    left = softmax_attention(h, w, p + "left.", m["left"], eps, positions)
    right = retention(h, w, p + "right.", m["right"], eps, positions)
    return 0.5 * (rms_norm(left, w[p + "left.out"], eps) + rms_norm(right, w[p + "right.out"], eps))


def lightning_mixer(h, w, p, m, eps):
    """silu maps for q, k, v; the decayed sum without any scale; all heads normed together,
    times sigmoid(gate)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(T, H, dk)
    k = silu(h @ w[p + "k"].T).reshape(T, H, dk)
    v = silu(h @ w[p + "v"].T).reshape(T, H, dv)
    o, _ = decayed_linear_attention(q, k, v, m["decay"])
    o = rms_norm(o.reshape(T, H * dv), w[p + "norm"], eps) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def expert(h, w, p, limit):
    """g = min(gate, limit), u = clamp(up, -limit, limit); down(g * sigmoid(1.702 g) * (u + 1))."""
    g = np.minimum(h @ w[p + "gate"].T, limit)
    u = np.clip(h @ w[p + "up"].T, -limit, limit)
    return (g * sigmoid(GATE_SLOPE * g) * (u + 1.0)) @ w[p + "down"].T


def router_logits(h, w, p):
    return h @ w[p + "router"].T + w[p + "router.b"]


def route(z, top):
    """(chosen [T, top], weights [T, top]): the largest logits, softmax over the chosen only."""
    order = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, order, axis=-1)
    e = np.exp(zc - zc.max(axis=-1, keepdims=True))
    return order, e / e.sum(axis=-1, keepdims=True)


def moe(h, w, p, m, forced=None, slack=0.0):
    """forced [T, top]: experts that another implementation chose. Where they differ from this
    function's own choice they must be as good within ``slack`` (a close call that rounding
    decides); the function then goes on with them."""
    T = h.shape[0]
    z = router_logits(h, w, p)
    top = m["router"]["top"]
    chosen, weight = route(z, top)
    if forced is not None:
        forced = np.asarray(forced, dtype=np.int64)
        for t in range(T):
            if set(forced[t]) != set(chosen[t]):
                assert len(set(forced[t])) == len(forced[t]), f"token {t}: an expert chosen twice"
                assert z[t, forced[t]].min() >= z[t, chosen[t]].min() - slack, \
                    f"token {t}: experts {forced[t]} chosen, {chosen[t]} have the largest logits: {z[t]}"
        zc = np.take_along_axis(z, forced, axis=-1)
        e = np.exp(zc - zc.max(axis=-1, keepdims=True))
        chosen, weight = forced, e / e.sum(axis=-1, keepdims=True)
    out = np.zeros((T, w[p + "e0.down"].shape[0]))
    limit = m["expert"]["limit"]
    for t in range(T):
        for e, g in zip(chosen[t], weight[t]):
            out[t] += g * expert(h[t][None], w, f"{p}e{int(e)}.", limit)[0]
    if m.get("shared") is not None:
        out += expert(h, w, p + "shared.", m["shared"]["limit"])
    return out


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainLuduvik:
    def __init__(self, folder=None, config=None, weights=None):
        if folder is not None:
            config = json.loads((Path(folder) / "config.json").read_text())
            weights = read_safetensors(Path(folder) / "model.safetensors")
        self.c, self.w = config, weights

    def forward(self, tokens, layers_out=None, routes=None, slack=0.03):
        """Logits [T, vocab] of a whole sequence from position 0. ``layers_out``: a list that
        receives the residual stream after every layer. ``routes``: {layer: experts [T, top]}
        chosen elsewhere (see ``moe``)."""
        c, w = self.c, self.w
        eps = c["norm"]["eps"]
        tokens = np.asarray(tokens, dtype=np.int64)
        positions = np.arange(len(tokens))
        x = np.array(w["embed"][tokens], dtype=np.float64)
        for li, layer in enumerate(c["layers"]):
            L, mx = f"l{li}.", layer["mixer"]
            h = rms_norm(x, w[L + "norm1"], eps)
            if layer["type"] == "parallel":
                out = parallel_mixer(h, w, L + "mix.", mx, eps, positions)
            elif layer["type"] == "lightning":
                out = lightning_mixer(h, w, L + "mix.", mx, eps)
            else:
                raise ValueError(f"layer {li}: unknown type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp["kind"] != "moe":
                    raise ValueError(f"layer {li}: unknown feed-forward {mlp['kind']!r}")
                out = out + moe(h, w, L + "mlp.", mlp, None if routes is None else routes.get(li), slack)
            x = x + out
            if layers_out is not None:
                layers_out.append(x.copy())
        return rms_norm(x, w["final.norm"], eps) @ w["head"].T

    def greedy(self, prompt, n):
        seq = list(prompt)
        for _ in range(n):
            seq.append(int(np.argmax(self.forward(seq)[-1])))
        return seq[len(prompt):]


# --------------------------------------------------------------------------
# random models for the tests
# --------------------------------------------------------------------------
def tensor_shapes(c):
    """{tensor name: shape} of a configuration, in the file's own names."""
    d, V = c["width"], c["vocab"]
    s = {"embed": (V, d), "final.norm": (d,), "head": (V, d)}
    for li, layer in enumerate(c["layers"]):
        L, mx, M = f"l{li}.", layer["mixer"], f"l{li}.mix."
        s[L + "norm1"] = (d,)
        if layer["type"] == "lightning":
            H, dk, dv = mx["heads"], mx["dim"], mx["vdim"]
            s[M + "q"], s[M + "k"] = (H * dk, d), (H * dk, d)
            s[M + "v"], s[M + "g"] = (H * dv, d), (H * dv, d)
            s[M + "o"], s[M + "norm"] = (d, H * dv), (H * dv,)
        else:
            a, r = mx["left"], mx["right"]
            A, R = M + "left.", M + "right."
            s[A + "q"] = (a["heads"] * a["dim"], d)
            s[A + "k"], s[A + "v"] = (a["kv_heads"] * a["dim"], d), (a["kv_heads"] * a["vdim"], d)
            s[A + "q.norm"], s[A + "k.norm"] = (a["dim"],), (a["dim"],)
            s[A + "o"] = (d, a["heads"] * a["vdim"])
            s[R + "q"], s[R + "k"] = (r["heads"] * r["dim"], d), (r["heads"] * r["dim"], d)
            s[R + "v"], s[R + "g"] = (r["heads"] * r["vdim"], d), (r["heads"] * r["vdim"], d)
            s[R + "o"] = (d, r["heads"] * r["vdim"])
            s[M + "left.out"], s[M + "right.out"] = (d,), (d,)
        mlp = layer.get("mlp")
        if mlp is not None:
            F, ff = L + "mlp.", mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                s[f"{F}e{e}.gate"], s[f"{F}e{e}.up"], s[f"{F}e{e}.down"] = (ff, d), (ff, d), (d, ff)
            s[F + "router"], s[F + "router.b"] = (mlp["router"]["experts"], d), (mlp["router"]["experts"],)
            if mlp.get("shared") is not None:
                ff = mlp["shared"]["ff"]
                s[F + "shared.gate"], s[F + "shared.up"], s[F + "shared.down"] = (ff, d), (ff, d), (d, ff)
    return s


def random_weights(c, seed, edit=None):
    """float64 weights, already rounded to bfloat16 values so that a bfloat16 file holds them
    exactly. Matrices ~ N(0, 1/sqrt(in)), gate and up maps twice that so that the experts'
    limits cut; gains near 1; router rows and biases large enough that the chosen experts are
    no close call."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(c).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm", "out"):
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif name.endswith("router"):
            a = 4.0 * rng.standard_normal(shape) / np.sqrt(shape[-1])
        elif name.endswith("router.b"):
            a = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            a = rng.standard_normal(shape)
        elif last in ("gate", "up"):
            a = 2.0 * rng.standard_normal(shape) / np.sqrt(shape[-1])
        else:
            a = rng.standard_normal(shape) / np.sqrt(shape[-1])
        w[name] = round_bf16(a)
    if edit is not None:
        edit(w)
        for n in w:
            w[n] = round_bf16(w[n].reshape(-1)).reshape(w[n].shape)
    return w


def make_model_folder(folder, c, seed, storage="BF16", edit=None):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    w = random_weights(c, seed, edit)
    write_safetensors(folder / "model.safetensors", w, dtype=storage)
    (folder / "config.json").write_text(json.dumps(c, indent=1))
    return w
