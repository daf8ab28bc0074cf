"""Saredra without a GPU: configuration keys, the layout it spells out, where parameters are
found in a file, binding errors, and the plain implementation's own invariants."""
import copy
import json

import numpy as np
import pytest

import plain_saredra as P
import saredra_util as U


def _cfg(d):
    from transformer_amd.config.saredra import SaredraConfig
    return SaredraConfig.from_dict(d)


def test_config_reads_every_key_and_writes_it_back():
    cfg = _cfg(U.CFG_A)
    assert (cfg.vocab, cfg.width, cfg.eps, len(cfg.layers)) == (211, 72, 1e-5, 5)
    l0 = cfg.layers[0]
    a, r, m = l0.left, l0.right, l0.mlp
    assert (l0.type, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.softcap, a.window, a.conv) == \
        ("parallel", 6, 2, 20, 12, 0.3, 5.0, 37, 3)
    assert (a.rot.dims, a.rot.base, a.rot.scaling) == (8, 300.0, (4.0, 64.0, 8.0, 1.0))
    assert (r.heads, r.vdim, r.state, r.groups, r.conv, r.norm_groups) == (4, 12, 10, 2, 2, 3)
    assert (l0.left_scale, l0.right_scale) == (1.3, 0.7)
    assert (m.kind, m.experts, m.top, m.ff, m.group_count, m.group_keep) == ("moe", 6, 2, 24, 3, 2)
    l1, l2 = cfg.layers[1], cfg.layers[2]
    assert (l1.type, l1.attention.kv_from, l1.mlp.kind, l1.mlp.ff) == ("attention", None, "dense", 40)
    assert (l2.attention.kv_from, l2.attention.window, l2.mlp) == (1, 20, None)
    assert (cfg.layers[3].mlp.group_count, cfg.layers[3].mlp.top) == (1, 4)
    assert _cfg(cfg.to_dict()) == cfg
    for c in (U.CFG_B, U.CFG_C, U.CFG_D):
        assert _cfg(_cfg(c).to_dict()) == _cfg(c)
    b = _cfg(U.CFG_B)            # absent keys: no window, no cap, no rotation, no convolution, scales of 1
    a0 = b.layers[0].attention
    assert (a0.window, a0.softcap, a0.rot, a0.conv) == (None, None, None, 0)
    assert (b.layers[1].left_scale, b.layers[1].right_scale, b.layers[2].left.conv) == (1.0, 1.0, 0)
    short = copy.deepcopy(U.CFG_B)       # as many kv heads as heads, values as wide as keys
    del short["layers"][0]["mixer"]["kv_heads"], short["layers"][0]["mixer"]["vdim"]
    assert (_cfg(short).layers[0].attention.kv_heads, _cfg(short).layers[0].attention.vdim) == (1, 32)


def test_config_errors_name_the_key():
    from transformer_amd.config.spec import ConfigError
    for path, value in ((("layers", 0, "type"), "mamba"), (("layers", 0, "mlp", "kind"), "glu"),
                        (("layers", 0, "mixer", "left", "kv_heads"), 4), (("layers", 0, "mixer", "left", "rot", "dims"), 7),
                        (("layers", 0, "mixer", "left", "rot", "dims"), 22), (("layers", 0, "mixer", "left", "mask", "size"), 0),
                        (("layers", 0, "mixer", "left", "softcap"), 0.0), (("layers", 0, "mixer", "right", "groups"), 3),
                        (("layers", 0, "mixer", "right", "norm_groups"), 5), (("layers", 0, "mixer", "right", "state"), None),
                        (("layers", 0, "mlp", "router", "top"), 5), (("layers", 0, "mlp", "router", "groups", "count"), 4),
                        (("layers", 0, "mlp", "router", "groups", "keep"), 4), (("layers", 1, "mlp", "ff"), 0),
                        (("layers", 2, "mixer", "kv_from"), 0), (("layers", 2, "mixer", "kv_from"), 2),
                        (("layers", 2, "mixer", "dim"), 18), (("layers", 4, "mixer", "kv_from"), 2),
                        (("layers", 0, "mixer", "left", "scale"), None), (("layers", 0, "mixer", "right"), None),
                        (("norm",), None), (("width",), 0), (("layers",), [])):
        d = copy.deepcopy(U.CFG_A)
        at = d
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            _cfg(d)


def test_layout_blocks_schedule_and_cache_needs():
    import math
    import torch
    from transformer_amd.cache.storage import KVNeed, StateNeed
    from transformer_amd.parts.base import build_part
    cfg = _cfg(U.CFG_A)
    spec = cfg.model_spec()
    assert [(r.block, r.cache_of) for r in spec.schedule] == [(0, None), (1, None), (2, 1), (3, None), (4, 1)]
    assert [b.kind for b in spec.blocks] == ["prenorm"] * 5
    assert [b.mixer.kind for b in spec.blocks] == ["branch_sum", "attention_sink", "attention_sink", "branch_sum", "attention_sink"]
    assert [b.ffn.kind if b.ffn is not None else None for b in spec.blocks] == ["routed_mlp", "glu", None, "routed_mlp", "routed_mlp"]
    assert spec.blocks[2].norm2 is None
    left, right = spec.blocks[0].mixer.branches
    assert spec.blocks[0].mixer.scales == (1.3, 0.7) and spec.blocks[0].mixer.names == ("left", "right")
    assert (left.sink, left.qkv_bias, left.conv_taps, left.out_gate, left.own_kv, left.softcap, left.window, left.rot_style) == \
        ("learned", True, 3, False, True, 5.0, 37, "interleaved")
    assert left.rot_ramp == (4.0, 64.0, 8.0, 1.0) and left.rot_magnitude == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert (right.kind, right.num_heads, right.head_dim, right.state, right.groups, right.taps, right.norm_groups) == \
        ("state_space", 4, 12, 10, 2, 2, 3)
    own, narrow, wide = spec.blocks[1].mixer, spec.blocks[2].mixer, spec.blocks[4].mixer
    assert (own.sink, own.qkv_bias, own.conv_taps, own.out_gate, own.own_kv, own.rot_magnitude) == ("unit", False, 0, True, True, 1.0)
    # the lender keeps its rows for the widest window among itself and its readers
    assert (own.window, narrow.window, wide.window) == (50, 20, 90)
    assert own.cache_window == narrow.cache_window == wide.cache_window == 90 == cfg.cache_window(1)
    assert not narrow.own_kv and not wide.own_kv
    f = spec.blocks[0].ffn
    assert (f.form, f.activation, f.score, f.renormalize, f.weight_on, f.shared_intermediate, f.groups, f.keep_groups) == \
        ("glu", "silu", "softmax", False, "output", None, 3, 2)
    needs = [build_part(b, torch.float32, "cpu").cache_need() for b in spec.blocks]
    assert needs[0] == [KVNeed(2, 20, 37, 12), StateNeed((2, 6 * 20 + 2 * 20 + 2 * 12)), StateNeed((4, 10, 12)), StateNeed((1, 48 + 40))]
    assert needs[1] == needs[2] == needs[4] == KVNeed(2, 16, 90, 24)
    b = _cfg(U.CFG_B).model_spec()       # no window: the cache keeps everything; one tap: no memory
    nb = [build_part(x, torch.float32, "cpu").cache_need() for x in b.blocks]
    assert nb[0] == KVNeed(1, 32, None, 32) and nb[1] == [KVNeed(1, 16, None, 16), StateNeed((1, 16, 64))]
    assert _cfg(U.CFG_D).cache_window(0) == 129
    free = copy.deepcopy(U.CFG_D)        # a reader that sees everything keeps its lender's rows for good
    del free["layers"][2]["mixer"]["mask"]
    fs = _cfg(free).model_spec()
    assert _cfg(free).cache_window(0) is None and (fs.blocks[0].mixer.window, fs.blocks[0].mixer.cache_window) == (65, 0)
    assert build_part(fs.blocks[0], torch.float32, "cpu").cache_need() == KVNeed(5, 6, None, 11) == \
        build_part(fs.blocks[2], torch.float32, "cpu").cache_need()
    assert spec.tie_embeddings is False and spec.after_embed is None and spec.on_logits is None


def test_every_parameter_has_a_file_tensor_and_back():
    from transformer_amd.config.registry import get_architecture
    from transformer_amd.engine.params import declared_params
    arch = get_architecture("Saredra")
    assert get_architecture("saredra") is arch
    for cfg_dict in (U.CFG_A, U.CFG_B, U.CFG_D):
        cfg = arch.config_from_dict(cfg_dict)
        params = declared_params(arch.model_spec(cfg))
        src = arch.weight_sources(cfg, "safetensors")
        assert set(src) == set(params)
        named = {}
        for pname, s in src.items():
            rows = sum(p.shape[0] for p in s.options[0])
            assert rows == params[pname].shape[0], pname
            named.update({p.name: p.shape for p in s.options[0]})
        assert named == {n: tuple(s) for n, s in P.tensor_shapes(cfg_dict).items()}


def test_loader_reports_missing_and_misshaped_tensors(tmp_path):
    from transformer_amd.api import open_model_source
    from transformer_amd.engine.params import declared_params
    from transformer_amd.weights.loader import WeightsError, plan_binding
    P.make_model_folder(tmp_path / "ok", U.CFG_A, 1)
    w = dict(P.random_weights(U.CFG_A, 1))
    arch, cfg, f = open_model_source(tmp_path / "ok")
    assert arch.name == "Saredra"
    plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    bad = dict(w)
    del bad["l0.mix.right.A_log"]
    bad["l0.mix.left.sink"] = bad["l0.mix.left.sink"][:-1]
    bad["l0.mix.left.k.conv"] = np.zeros((40, 4))
    bad["l2.mix.k"] = np.zeros((32, 72))            # a reader has no keys of its own
    (tmp_path / "bad").mkdir()
    P.write_safetensors(tmp_path / "bad" / "model.safetensors", bad, "BF16")
    (tmp_path / "bad" / "config.json").write_text(json.dumps(U.CFG_A))
    arch, cfg, f = open_model_source(tmp_path / "bad")
    with pytest.raises(WeightsError) as e:
        plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    assert e.value.missing == ["l0.mix.right.A_log"] and e.value.unexpected == ["l2.mix.k"]
    assert sorted(n for n, _, _ in e.value.wrong_shape) == ["l0.mix.left.k.conv", "l0.mix.left.sink"]


def test_ramp_frequencies_of_the_product_match_the_plain_ones():
    from transformer_amd.parts.position import ramp_frequencies
    for dims, base, sc in ((8, 300.0, (4.0, 64, 8.0, 1.0)), (64, 5e5, (4.0, 2048, 32.0, 1.0)), (34, 20.0, (3.0, 40, 6.0, 2.0)),
                           (2, 7.0, (2.0, 4, 8.0, 0.5)), (24, 50.0, (2.0, 32, 4.0, 0.5))):
        rot = U._rot(dims, base, sc)
        np.testing.assert_allclose(ramp_frequencies(dims, base, sc), P.rotation_frequencies(rot)[0], rtol=1e-13)


# ---------------------------------------------------------------- the plain functions themselves
def test_plain_frequencies_keep_fast_and_slow_the_rest():
    rot = U._rot(8, 300.0, (4.0, 64, 8.0, 1.0))
    f = 300.0 ** (-np.arange(4) / 4.0)
    got, mag = P.rotation_frequencies(rot)
    n = lambda t: 8 * np.log(64 / (2 * np.pi * t)) / (2 * np.log(300.0))
    assert 0 < n(8.0) < 1 and 1 < n(1.0) < 2                       # lo = 0, hi = 2: pair 0 kept, 1 half, 2 and 3 slowed
    np.testing.assert_allclose(got, [f[0], 0.5 * f[1] / 4 + 0.5 * f[1], f[2] / 4, f[3] / 4])
    assert mag == pytest.approx(0.1 * np.log(4.0) + 1.0)
    plain, one = P.rotation_frequencies(U._rot(8, 300.0))
    np.testing.assert_allclose(plain, f)
    assert one == 1.0


def test_plain_rotation_pairs_neighbours_and_keeps_relative_angles():
    rng = np.random.default_rng(0)
    t = rng.standard_normal((5, 2, 12))
    rot = U._rot(8, 100.0)
    r = P.rotate_pairs(t, np.arange(5), rot)
    np.testing.assert_allclose(r[..., 8:], t[..., 8:])
    np.testing.assert_allclose(np.linalg.norm(r, axis=-1), np.linalg.norm(t, axis=-1))
    np.testing.assert_allclose(r[0], t[0])
    one = np.zeros((2, 1, 4))
    one[:, 0, 0] = 1.0                                     # coordinate 0 turns into coordinate 1, not 2
    np.testing.assert_allclose(P.rotate_pairs(one, [0, 1], U._rot(4, 10.0))[1, 0], [np.cos(1.0), np.sin(1.0), 0, 0])
    a = P.rotate_pairs(t, np.arange(5) + 9, rot)
    np.testing.assert_allclose(np.einsum("thd,shd->tsh", a, a), np.einsum("thd,shd->tsh", r, r), atol=1e-9)
    big = P.rotate_pairs(t, np.arange(5), U._rot(12, 100.0, (2.0, 16, 4.0, 1.0)))      # the magnitude scales rotated pairs
    np.testing.assert_allclose(np.linalg.norm(big, axis=-1), np.linalg.norm(t, axis=-1) * (0.1 * np.log(2.0) + 1.0))


def test_plain_convolution_carries_its_inputs():
    rng = np.random.default_rng(1)
    u, w, b = rng.standard_normal((9, 3)), rng.standard_normal((3, 4)), rng.standard_normal(3)
    whole = P.causal_conv(u, w, b)
    np.testing.assert_allclose(whole[0], w[:, 3] * u[0] + b)                   # the last column is the current token's
    np.testing.assert_allclose(whole[2], w[:, 1] * u[0] + w[:, 2] * u[1] + w[:, 3] * u[2] + b)
    second = P.causal_conv(u[5:], w, b, before=u[2:5])
    np.testing.assert_allclose(second, whole[5:])
    np.testing.assert_allclose(P.causal_conv(u, w[:, :1]), u * w[:, 0])       # one tap: no memory


def test_plain_softmax_window_cap_and_sink():
    rng = np.random.default_rng(2)
    T, H, G, dk, dv = 12, 4, 2, 6, 3
    q, k, v = rng.standard_normal((T, H, dk)), rng.standard_normal((T, G, dk)), rng.standard_normal((T, G, dv))
    full = P.windowed_softmax_attention(q, k, v, 0.4)
    np.testing.assert_allclose(full[0], np.repeat(v[0], 2, axis=0))           # the first token sees itself only
    np.testing.assert_allclose(P.windowed_softmax_attention(q, k, v, 0.4, window=T), full)
    one = P.windowed_softmax_attention(q, k, v, 0.4, window=1)
    np.testing.assert_allclose(one, np.repeat(v, 2, axis=1))
    w3 = P.windowed_softmax_attention(q, k, v, 0.4, window=3)
    np.testing.assert_allclose(w3[7], P.windowed_softmax_attention(q[5:8], k[5:8], v[5:8], 0.4)[2])   # 5, 6, 7 and no more
    sunk = P.windowed_softmax_attention(q, k, v, 0.4, window=1, sink=np.array([0.0, -50.0, 50.0, np.log(3.0)]))
    np.testing.assert_allclose(sunk[:, 1], one[:, 1])
    np.testing.assert_allclose(sunk[:, 2], 0.0, atol=1e-12)
    s = np.einsum("thd,thd->th", q, np.repeat(k, 2, axis=1)) * 0.4
    np.testing.assert_allclose(sunk[:, 0], one[:, 0] * (np.exp(s[:, 0]) / (1 + np.exp(s[:, 0])))[:, None])
    np.testing.assert_allclose(sunk[:, 3], one[:, 3] * (np.exp(s[:, 3]) / (3 + np.exp(s[:, 3])))[:, None])
    capped = P.windowed_softmax_attention(100 * q, k, v, 0.4, softcap=1e-3)    # a tiny cap flattens the weights
    np.testing.assert_allclose(capped[5], np.repeat(v[:6].mean(0), 2, axis=0), atol=2e-3)


def test_plain_state_space_equals_its_sum_form_and_carries_its_state():
    rng = np.random.default_rng(3)
    T, H, Pd, N, G = 11, 4, 3, 5, 2
    x, B, C = rng.standard_normal((T, H, Pd)), rng.standard_normal((T, G, N)), rng.standard_normal((T, G, N))
    dt, a_log, D = rng.uniform(0.1, 2.0, (T, H)), rng.uniform(-2, 1, H), rng.standard_normal(H)
    got, S = P.selective_scan(x, B, C, dt, a_log, D, G)
    np.testing.assert_allclose(got, P.selective_scan_sum(x, B, C, dt, a_log, D, G), atol=1e-12)
    a, S1 = P.selective_scan(x[:4], B[:4], C[:4], dt[:4], a_log, D, G)
    b, S2 = P.selective_scan(x[4:], B[4:], C[4:], dt[4:], a_log, D, G, S1)
    np.testing.assert_allclose(np.concatenate([a, b]), got, atol=1e-12)
    np.testing.assert_allclose(S2, S, atol=1e-12)
    np.testing.assert_allclose(got[0, 3], dt[0, 3] * (B[0, 1] @ C[0, 1]) * x[0, 3] + D[3] * x[0, 3])     # head 3 reads group 1
    y = rng.standard_normal((2, 12))
    n = P.grouped_unit_rms(y, 3, 0.0)
    np.testing.assert_allclose((n.reshape(2, 3, 4) ** 2).mean(-1), 1.0)


def test_plain_routing_in_groups_and_close_calls():
    s = np.array([0.05, 0.30, 0.28, 0.02, 0.20, 0.15])
    assert list(P.route(s, 2)) == [1, 2]
    assert list(P.route(s, 2, 3, 1)) == [1, 0]                   # the best group alone: experts 0 and 1
    assert list(P.route(s, 3, 3, 2)) == [1, 2, 0]                # groups (0, 1) and (2, 3)
    assert list(P.route(s, 2, 2, 1)) == [1, 2]
    assert list(P.route(np.full(4, 0.25), 2, 2, 1)) == [0, 1]    # the lowest index among equals
    assert P.close_call(s, [1, 0], 2, 3, 1, 0.0) and not P.close_call(s, [2, 3], 2, 3, 1, 0.01)
    assert P.close_call(s, [2, 3], 2, 3, 1, 0.03)                # group (2, 3) is within 0.03 of the best
    assert not P.close_call(s, [1, 4], 2, 3, 1, 0.03) and not P.close_call(s, [1, 1], 2, 3, 1, 1.0)
    assert P.close_call(s, [1, 4], 2, 1, 1, 0.09) and not P.close_call(s, [1, 4], 2, 1, 1, 0.07)
    w = {"router": np.log(s)[:, None] * np.ones((1, 2)) / 2}
    for e in range(6):
        w.update({f"e{e}.gate": np.ones((1, 2)), f"e{e}.up": np.full((1, 2), float(e)), f"e{e}.down": np.ones((2, 1))})
    m = {"router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}, "expert": {"ff": 1}}
    out, chosen = P.moe(np.ones((1, 2)), w, "", m)
    assert list(chosen[0]) == [1, 0]
    np.testing.assert_allclose(out[0], (0.30 * 1 + 0.05 * 0) * P.silu(2.0) * 2.0 * np.ones(2))        # the scores themselves


def test_plain_model_is_causal_and_adds_its_sublayers_in_turn():
    m = U.plain("B", "float32")
    toks = U.tokens("B", 12, 0)
    a, b = m.forward(toks)[0], m.forward(toks[:7])[0]
    np.testing.assert_allclose(a[:7], b, atol=1e-10)
    _, layers = m.forward(toks[:3])
    w, eps, c = m.w, m.eps, m.c
    x0 = w["embed"][toks[:3]]
    x1 = x0 + P.gated_attention(P.rms_norm(x0, w["l0.norm1"], eps), w, "l0.mix.", c["layers"][0]["mixer"], np.arange(3))[0]
    want = x1 + P.moe(P.rms_norm(x1, w["l0.norm2"], eps), w, "l0.mlp.", c["layers"][0]["mlp"])[0]
    np.testing.assert_allclose(layers[0], want, atol=1e-12)
    h = P.rms_norm(layers[0], w["l1.norm1"], eps)          # a layer without a feed-forward adds its mixer alone
    np.testing.assert_allclose(layers[1], layers[0] + P.parallel_mixer(h, w, "l1.mix.", c["layers"][1]["mixer"], eps, np.arange(3)),
                               atol=1e-12)


def test_bench_shapes_of_the_design_option_are_valid_models():
    import bench
    import transformer_amd as ta
    for size, (base, kinds, near) in bench.saredra_shapes().items():
        for kind, layers in kinds.items():
            cfg = ta.SaredraConfig.from_dict({**base, "layers": layers})
            spec = cfg.model_spec()
            assert len(spec.blocks) == len(layers) and spec.hidden == base["width"], (size, kind)
        assert [r.cache_of for r in ta.SaredraConfig.from_dict({**base, "layers": kinds["mixed"]}).model_spec().schedule] == \
            [None, None, 0, None]
        for arch, cfg_dict in near.values():
            assert ta.get_architecture(arch).config_from_dict(cfg_dict).model_spec().hidden == base["width"]
