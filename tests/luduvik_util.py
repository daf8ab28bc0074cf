"""Tiny Luduvik configurations and helpers shared by the Luduvik tests. Sizes differ between the
configurations and from one another inside each (heads and kv heads, key and value widths of
both branches, rotated coordinates, experts and their widths), few are powers of two, and the
corners (one head, one kv head, as many kv heads as heads, one expert, as many chosen as there
are, no shared expert, no feed-forward, no rotation, no frequency scaling, a rotation of whole
heads and of a part, decays of 0 and 1) each appear somewhere."""
import functools
import tempfile

import numpy as np

import plain_luduvik as P


def _rot(dims, base, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def _left(heads, kv_heads, dim, vdim, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        m["rot"] = rot
    return m


def _lin(heads, dim, vdim, decay, rot=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot is not None:
        m["rot"] = rot
    return m


def _moe(experts, top, ff, limit, shared=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared is not None:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def _par(left, right, mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def _lit(lin, mlp=None):
    return {"type": "lightning", "mixer": lin, "mlp": mlp}


# a parallel layer first; three query heads per kv head, values narrower than keys and wider;
# scaled frequencies whose three regimes (kept, slowed, blended) all occur among four pairs;
# two and three chosen experts, all of them chosen, no shared expert, no feed-forward
CFG_A = {
    "architecture": "Luduvik", "vocab": 211, "width": 72, "norm": {"eps": 1e-5},
    "layers": [
        _par(_left(6, 2, 20, 12, 0.3, _rot(8, 1000.0, (8.0, 1.0, 4.0, 64))),
             _lin(3, 12, 20, [0.9, 0.99, 0.5], _rot(12, 100.0)), _moe(5, 2, 24, 1.0, shared=(40, 0.7))),
        _lit(_lin(3, 8, 24, [0.97, 0.8, 0.999]), _moe(3, 3, 16, 2.0)),
        _lit(_lin(1, 40, 16, [0.95])),
        _par(_left(4, 4, 16, 24, 0.25), _lin(2, 16, 8, [0.6, 0.995], _rot(4, 50.0)), _moe(7, 1, 20, 0.5, shared=(12, 3.0))),
        _lit(_lin(5, 4, 4, [0.9, 0.9, 0.2, 1.0, 0.0]), _moe(4, 2, 8, 1.5, shared=(8, 1.5))),
    ],
}
# the corners: one head and one kv head, one expert, whole heads rotated without scaling, a
# lightning layer first and last, a retention branch without any rotation
CFG_B = {
    "architecture": "Luduvik", "vocab": 50, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        _lit(_lin(1, 64, 64, [0.98]), _moe(1, 1, 32, 1.0, shared=(8, 1.0))),
        _par(_left(1, 1, 16, 16, 0.25, _rot(16, 10000.0)), _lin(1, 16, 16, [0.9])),
        _par(_left(4, 1, 8, 40, 0.4, _rot(2, 300.0)), _lin(4, 8, 8, [0.5, 0.7, 0.9, 0.99], _rot(8, 300.0, (2.0, 1.0, 2.0, 16))),
             _moe(4, 2, 8, 0.8)),
        _lit(_lin(2, 24, 12, [1.0, 0.9])),
    ],
}
# wide enough for the matrix cores: heads of 128 with narrower values and heads of 64 with
# equal ones (both take the matrix-core attention), experts on the matrix cores, products that
# leave planes
CFG_C = {
    "architecture": "Luduvik", "vocab": 1200, "width": 1024, "norm": {"eps": 1e-5},
    "layers": [
        _lit(_lin(16, 64, 64, [1.0 - 2.0 ** -(3 + i / 2) for i in range(16)]), _moe(8, 2, 256, 1.5, shared=(512, 1.0))),
        _par(_left(8, 2, 128, 64, 0.09, _rot(64, 50000.0, (4.0, 1.0, 4.0, 256))),
             _lin(8, 128, 128, [1.0 - 2.0 ** -(4 + i) for i in range(8)], _rot(128, 50000.0)), _moe(6, 3, 128, 1.2, shared=(256, 2.0))),
        _par(_left(16, 4, 64, 64, 0.125, _rot(32, 10000.0)), _lin(4, 96, 160, [0.9, 0.99, 0.999, 0.9999], _rot(32, 10000.0))),
    ],
}
# a width that is no multiple of four, odd sizes everywhere
CFG_D = {
    "architecture": "Luduvik", "vocab": 77, "width": 90, "norm": {"eps": 1e-5},
    "layers": [
        _lit(_lin(3, 14, 10, [0.9, 0.8, 0.7]), _moe(9, 4, 10, 1.0, shared=(3, 0.5))),
        _par(_left(5, 5, 7, 11, 0.35, _rot(6, 100.0)), _lin(2, 33, 5, [0.93, 0.999], _rot(2, 100.0)), _moe(2, 1, 33, 4.0)),
        _par(_left(2, 1, 34, 6, 0.2, _rot(34, 20.0, (3.0, 1.0, 3.0, 32))), _lin(3, 6, 22, [0.99, 0.5, 0.9])),
    ],
}
CONFIGS = {"A": (CFG_A, 31), "B": (CFG_B, 32), "C": (CFG_C, 33), "D": (CFG_D, 34)}
STORAGE = {"float32": "F32", "bfloat16": "BF16"}
# a bfloat16 engine may choose another expert than the plain model where the two logits are this
# close (the logits spread over several units; rounding of the rows in front of the router moves
# them by up to a tenth)
SLACK = 0.15
# largest allowed rms(engine - plain) / rms(plain) over a row of logits
TOL = {"float32": 2e-4, "bfloat16": 1e-1}

_keep = []


def _sharp(w):
    """Peaked softmax: larger query and key gains make one key stand out, so a fault in any
    single key (a far one, one at a page's border, one of the wrong position) moves the logits."""
    for n in w:
        if n.endswith("left.q.norm") or n.endswith("left.k.norm"):
            w[n] = w[n] * 3.0


EDITS = {None: None, "sharp": _sharp}


@functools.lru_cache(maxsize=None)
def folder(name, dtype, edit=None):
    cfg, seed = CONFIGS[name]
    d = tempfile.TemporaryDirectory(prefix=f"lu_{name}_{dtype}_")
    _keep.append(d)
    P.make_model_folder(d.name, cfg, seed, storage=STORAGE[dtype], edit=EDITS[edit])
    return d.name


@functools.lru_cache(maxsize=None)
def plain(name, dtype, edit=None):
    return P.PlainLuduvik(folder(name, dtype, edit))


@functools.lru_cache(maxsize=None)
def engine(name, dtype, edit=None):
    import transformer_amd as ta
    return ta.load_model(folder(name, dtype, edit), dtype, "cuda:0")


def tokens(name, n, seed):
    cfg, _ = CONFIGS[name]
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


@functools.lru_cache(maxsize=None)
def plain_logits(name, dtype, edit, toks):
    return plain(name, dtype, edit).forward(list(toks))


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
    was a close call indeed, and follows it (``plain_luduvik.moe``). Steps run eagerly meanwhile."""

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
        want = plain(name, dtype, edit).forward(list(toks), routes=routes, slack=SLACK)
    err = row_error(got, want[:len(got)]).max()
    assert err < TOL[dtype], f"{what}: {err}"
