"""Tiny Saredra configurations and helpers shared by the Saredra tests. Sizes differ between the
configurations and from one another inside each (heads and kv heads, key and value widths,
rotated coordinates, windows, taps, state sizes, groups of experts), few are powers of two, and the
corners (one head, one kv head, as many kv heads as heads, one expert, all experts chosen, one
group, every group kept, no window, no cap, no rotation, no slowed frequencies, one tap, no
convolution, no feed-forward, a reader whose window is wider than its lender's) each appear
somewhere."""
import functools
import tempfile

import numpy as np

import plain_saredra as P


def _rot(dims, base, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _heads(heads, kv_heads, dim, vdim, scale, window=None, softcap=None, rot=None, conv=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if softcap is not None:
        m["softcap"] = softcap
    if rot is not None:
        m["rot"] = rot
    if conv is not None:
        m["conv"] = conv
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, groups=None):
    r = {"experts": experts, "top": top}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": r, "expert": {"ff": ff}}


def _att(heads, mlp=None):
    return {"type": "attention", "mixer": heads, "mlp": mlp}


def _par(left, right, scales=(1.0, 1.0), mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": scales[0], "right": right, "right_scale": scales[1]},
            "mlp": mlp}


# a parallel layer first; three query heads per kv head; values narrower than keys and wider; slowed
# frequencies whose ramp lies inside the pairs; windows shorter than a page and longer; a reader with
# a narrower and one with a wider window than its lender; three groups of experts of which two stay
CFG_A = {
    "architecture": "Saredra", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
    "layers": [
        _par(_heads(6, 2, 20, 12, 0.3, 37, 5.0, _rot(8, 300.0, (4.0, 64, 8.0, 1.0)), conv=3), _ssm(4, 12, 10, 2, 2, 3),
             (1.3, 0.7), _moe(6, 2, 24, (3, 2))),
        _att(_heads(4, 2, 16, 24, 0.25, 50, 8.0, _rot(6, 1000.0)), _dense(40)),
        _att(_heads(4, 2, 16, 24, 0.2, 20, 4.0, _rot(6, 1000.0), kv_from=1)),
        _par(_heads(2, 1, 24, 8, 0.2, 70, 20.0, _rot(24, 50.0, (2.0, 32, 4.0, 0.5)), conv=5), _ssm(3, 8, 6, 3, 4, 1),
             (0.8, 1.1), _moe(4, 4, 16)),
        _att(_heads(4, 2, 16, 24, 0.3, 90, 30.0, _rot(6, 1000.0), kv_from=1), _moe(5, 1, 20)),
    ],
}
# the corners: one head and one kv head, one expert, no window, no cap, no rotation, one tap and no
# convolution at all, one group of state-space heads and as many as heads, scales left at 1
CFG_B = {
    "architecture": "Saredra", "vocab": 50, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        _att(_heads(1, 1, 32, 32, 0.18), _moe(1, 1, 32)),
        {"type": "parallel", "mixer": {"left": _heads(1, 1, 16, 16, 0.25, rot=_rot(16, 10000.0), conv=1),
                                       "right": _ssm(1, 64, 16, 1, 1, 1)}, "mlp": None},
        _par(_heads(4, 4, 8, 40, 0.4, 3, 2.0, _rot(2, 300.0)), _ssm(4, 6, 40, 4, 3, 2), (2.0, 0.5), _moe(4, 2, 8, (2, 2))),
        _att(_heads(4, 1, 8, 2, 0.4, 1, None, _rot(8, 20.0, (8.0, 16, 2.0, 1.0))), _dense(24)),
    ],
}
# wide enough for the library's products of many rows and the experts' matrix-core products: heads of
# 128 with narrower values, 64 state-space heads' worth of columns, windows of several pages
CFG_C = {
    "architecture": "Saredra", "vocab": 1200, "width": 1024, "norm": {"eps": 1e-5},
    "layers": [
        _att(_heads(8, 2, 128, 64, 0.09, 200, 50.0, _rot(64, 50000.0)), _dense(1408)),
        _par(_heads(16, 4, 64, 64, 0.125, 130, 30.0, _rot(32, 10000.0, (2.0, 512, 16.0, 1.0)), conv=4),
             _ssm(16, 64, 64, 2, 4, 4), (1.2, 0.9), _moe(8, 2, 256, (4, 2))),
        _att(_heads(8, 2, 128, 64, 0.09, 300, 50.0, _rot(64, 50000.0), kv_from=0), _moe(6, 3, 128, (2, 1))),
    ],
}
# a width that is no multiple of four, odd sizes everywhere
CFG_D = {
    "architecture": "Saredra", "vocab": 77, "width": 90, "norm": {"eps": 1e-5},
    "layers": [
        _att(_heads(5, 5, 6, 11, 0.35, 65, 3.0, _rot(6, 100.0)), _moe(9, 4, 10, (3, 3))),
        _par(_heads(3, 1, 34, 7, 0.2, 64, 9.0, _rot(34, 20.0, (3.0, 40, 6.0, 2.0)), conv=2), _ssm(5, 7, 33, 1, 6, 5),
             (0.5, 1.5), _dense(33)),
        _att(_heads(5, 5, 6, 11, 0.3, 129, None, _rot(6, 100.0), kv_from=0)),
    ],
}
CONFIGS = {"A": (CFG_A, 41), "B": (CFG_B, 42), "C": (CFG_C, 43), "D": (CFG_D, 44)}
STORAGE = {"float32": "F32", "bfloat16": "BF16"}
# a bfloat16 engine may choose another expert than the plain model where the two scores are this
# close (rounding of the rows in front of the router moves the logits by up to a tenth)
SLACK = 0.06
# largest allowed rms(engine - plain) / rms(plain) over a row of logits
TOL = {"float32": 2e-4, "bfloat16": 1e-1}

_keep = []


def _sharp(w):
    """Peaked softmax: larger queries make one key stand out, so a fault in any single key (a far
    one, one at a page's or a window's border, one of the wrong position) moves the logits."""
    for n in list(w):
        if n.endswith("mix.q") or n.endswith("left.q"):
            w[n] = w[n] * 6.0


EDITS = {None: None, "sharp": _sharp}


@functools.lru_cache(maxsize=None)
def folder(name, dtype, edit=None):
    cfg, seed = CONFIGS[name]
    d = tempfile.TemporaryDirectory(prefix=f"sa_{name}_{dtype}_")
    _keep.append(d)
    P.make_model_folder(d.name, cfg, seed, storage=STORAGE[dtype], edit=EDITS[edit])
    return d.name


@functools.lru_cache(maxsize=None)
def plain(name, dtype, edit=None):
    return P.PlainSaredra(folder(name, dtype, edit))


@functools.lru_cache(maxsize=None)
def engine(name, dtype, edit=None):
    import transformer_amd as ta
    return ta.load_model(folder(name, dtype, edit), dtype, "cuda:0")


def tokens(name, n, seed):
    cfg, _ = CONFIGS[name]
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


@functools.lru_cache(maxsize=None)
def plain_logits(name, dtype, edit, toks):
    return plain(name, dtype, edit).forward(list(toks))[0]


def row_error(got, want):
    """rms of the difference (mean taken off) over rms of the expected row, per row."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(axis=-1, keepdims=True)
    return np.sqrt((d ** 2).mean(axis=-1)) / np.sqrt((want ** 2).mean(axis=-1))


class Routes:
    """Collects the experts that the engine's routed feed-forwards choose, step by step:
    ``with Routes(model) as r`` ... ``r.steps`` is a list of {layer: [tokens of the step, top]}.
    A bfloat16 engine decides a close call between two experts differently from the float64
    plain model now and then; the plain model is then told the engine's choice, checks that it
    was a close call indeed, and follows it (``plain_saredra.moe``). Steps run eagerly meanwhile."""

    def __init__(self, model):
        self.model, self.steps = model, []

    def __enter__(self):
        self.steps.append({})
        self.model.dump = self._take
        return self

    def __exit__(self, *exc):
        self.model.dump = None
        return False

    def _take(self, name, t):
        if name.endswith(".experts"):
            self.steps[-1][int(name.split(".")[1])] = t.detach().cpu().numpy().copy()

    def next_step(self):
        self.steps.append({})

    def of_rows(self, rows_of_step):
        """{layer: [T, top]} of one sequence: rows_of_step[i] = slice of its rows in step i (or None)."""
        out = {}
        for step, rows in zip(self.steps, rows_of_step):
            if rows is None:
                continue
            for layer, chosen in step.items():
                out.setdefault(layer, []).append(chosen[rows])
        return {layer: np.concatenate(parts) for layer, parts in out.items()}


def run_cuts(model, cache, slot, toks, cuts, routes=False):
    """Feeds ``toks`` into ``slot`` in portions of the given sizes (the rest one by one) and
    returns the logits of every position, [len(toks), vocab]; with ``routes`` also the experts
    the engine chose, {layer: [len(toks), top]}."""
    from transformer_amd import Entry
    out, at = [], 0
    sizes = list(cuts)
    rec = Routes(model) if routes else None
    if rec is not None:
        rec.__enter__()
    try:
        while at < len(toks):
            n = sizes.pop(0) if sizes else 1
            n = min(n, len(toks) - at)
            lg = model.step(cache, [Entry(slot, toks[at:at + n], list(range(n)))])
            out.append(lg.detach().cpu().numpy().copy())
            at += n
            if rec is not None:
                rec.next_step()
    finally:
        if rec is not None:
            rec.__exit__()
    logits = np.concatenate(out, 0)
    if rec is None:
        return logits
    return logits, rec.of_rows([slice(None)] * len(rec.steps))


def check_against_plain(name, dtype, edit, toks, got, routes=None, what=""):
    """The engine's logits of a whole sequence against the plain model's. float32: the plain
    model's own routing, every row. bfloat16: the plain model follows the engine's choice of
    experts where that was a close call (and fails where it was not)."""
    toks = list(toks)[:len(got)]
    if dtype == "float32" or not routes:
        want = plain_logits(name, dtype, edit, tuple(toks))
    else:
        want = plain(name, dtype, edit).forward(list(toks), forced=routes, slack=SLACK)[0]
    err = row_error(got, want[:len(got)]).max()
    assert err < TOL[dtype], f"{what}: {err}"
