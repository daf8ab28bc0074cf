"""Luduvik without a GPU: configuration keys, the layout it spells out, where parameters are
found in a file, binding errors, and the plain implementation's own invariants."""
import copy
import json

import numpy as np
import pytest

import luduvik_util as U
import plain_luduvik as P


def _cfg(d):
    from transformer_amd.config.luduvik import LuduvikConfig
    return LuduvikConfig.from_dict(d)


def test_config_reads_every_key_and_writes_it_back():
    cfg = _cfg(U.CFG_A)
    assert (cfg.vocab, cfg.width, cfg.eps, len(cfg.layers)) == (211, 72, 1e-5, 5)
    l0 = cfg.layers[0]
    a, r, m = l0.left, l0.right, l0.mlp
    assert (l0.type, a.heads, a.kv_heads, a.dim, a.vdim, a.scale) == ("parallel", 6, 2, 20, 12, 0.3)
    assert (a.rot.dims, a.rot.base, a.rot.scaling) == (8, 1000.0, (8.0, 1.0, 4.0, 64.0))
    assert (r.heads, r.dim, r.vdim, r.decay, r.rot.dims, r.rot.base, r.rot.scaling) == \
        (3, 12, 20, (0.9, 0.99, 0.5), 12, 100.0, None)
    assert (m.experts, m.top, m.ff, m.limit, m.shared_ff, m.shared_limit) == (5, 2, 24, 1.0, 40, 0.7)
    l1 = cfg.layers[1]
    assert (l1.type, l1.lightning.heads, l1.lightning.dim, l1.lightning.vdim, l1.lightning.rot) == ("lightning", 3, 8, 24, None)
    assert l1.mlp.shared_ff is None and l1.mlp.top == 3 and cfg.layers[2].mlp is None
    assert cfg.layers[3].left.rot is None and cfg.layers[3].left.kv_heads == 4
    assert _cfg(cfg.to_dict()) == cfg
    for c in (U.CFG_B, U.CFG_C, U.CFG_D):
        assert _cfg(_cfg(c).to_dict()) == _cfg(c)
    short = copy.deepcopy(U.CFG_B)                       # absent keys: as many kv heads as heads, values as wide as keys
    del short["layers"][1]["mixer"]["left"]["kv_heads"], short["layers"][1]["mixer"]["left"]["vdim"]
    del short["layers"][3]["mixer"]["vdim"]
    c = _cfg(short)
    assert (c.layers[1].left.kv_heads, c.layers[1].left.vdim, c.layers[3].lightning.vdim) == (1, 16, 24)


def test_config_errors_name_the_key():
    from transformer_amd.config.spec import ConfigError
    for path, value in ((("layers", 0, "type"), "mamba"), (("layers", 0, "mlp", "kind"), "glu"),
                        (("layers", 0, "mixer", "left", "kv_heads"), 4), (("layers", 0, "mixer", "left", "rot", "dims"), 7),
                        (("layers", 0, "mixer", "left", "rot", "dims"), 22), (("layers", 0, "mixer", "right", "decay"), [0.5, 0.5]),
                        (("layers", 1, "mixer", "decay"), [0.5, 0.5, 1.5]), (("layers", 1, "mixer", "decay"), None),
                        (("layers", 0, "mlp", "router", "top"), 6), (("layers", 0, "mlp", "expert", "limit"), 0.0),
                        (("layers", 0, "mlp", "shared", "limit"), -1.0), (("layers", 0, "mixer", "left", "scale"), None),
                        (("layers", 0, "mixer", "right"), None), (("norm",), None), (("width",), 0), (("layers",), [])):
        d = copy.deepcopy(U.CFG_A)
        at = d
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            _cfg(d)


def test_layout_blocks_and_cache_needs():
    import torch
    from transformer_amd.cache.storage import KVNeed, StateNeed
    from transformer_amd.parts.base import build_part
    spec = _cfg(U.CFG_A).model_spec()
    assert [r.block for r in spec.schedule] == [0, 1, 2, 3, 4] and all(r.cache_of is None for r in spec.schedule)
    assert [b.kind for b in spec.blocks] == ["parallel_prenorm"] * 5
    assert [b.mixer.kind for b in spec.blocks] == ["branch_mean", "decay_linear_attention", "decay_linear_attention",
                                                  "branch_mean", "decay_linear_attention"]
    assert [b.ffn.kind if b.ffn is not None else None for b in spec.blocks] == \
        ["routed_mlp", "routed_mlp", None, "routed_mlp", "routed_mlp"]
    left, right = spec.blocks[0].mixer.branches
    assert (left.kind, left.qk_norm_per_head, left.rot_dims, left.rot_scaling, left.scale, left.window) == \
        ("attention_normed", True, 8, (8.0, 1.0, 4.0, 64.0), 0.3, None)
    assert (right.key_scale, right.head_norm, right.norm_weight, right.gate_activation, right.input_activation, right.rot_dims) == \
        (12 ** -0.5, "per_head", False, "silu", None, 12)
    light = spec.blocks[1].mixer
    assert (light.key_scale, light.head_norm, light.norm_weight, light.gate_activation, light.input_activation, light.rot_dims) == \
        (1.0, "all_heads", True, "sigmoid", "silu", 0)
    f = spec.blocks[0].ffn
    assert (f.form, f.score, f.renormalize, f.weight_on, f.router_bias, f.shared_gate, f.limit, f.shared_limit, f.gate_slope,
            f.up_shift) == ("limited_glu", "softmax", True, "output", True, False, 1.0, 0.7, 1.702, 1.0)
    needs = [build_part(b, torch.float32, "cpu").cache_need() for b in spec.blocks]
    assert needs[0] == [KVNeed(2, 20, None, 12), StateNeed((3, 12, 20))]
    assert needs[1] == StateNeed((3, 8, 24)) and needs[2] == StateNeed((1, 40, 16))
    assert needs[3] == [KVNeed(4, 16, None, 24), StateNeed((2, 16, 8))]
    assert spec.tie_embeddings is False and spec.after_embed is None and spec.on_logits is None


def test_every_parameter_has_a_file_tensor_and_back():
    from transformer_amd.config.registry import get_architecture
    from transformer_amd.engine.params import declared_params
    arch = get_architecture("Luduvik")
    assert get_architecture("luduvik") is arch
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
    w = P.make_model_folder(tmp_path / "ok", U.CFG_B, 1)
    arch, cfg, f = open_model_source(tmp_path / "ok")
    assert arch.name == "Luduvik"
    plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    bad = dict(w)
    del bad["l1.mix.right.out"]
    bad["l1.mix.left.q.norm"] = bad["l1.mix.left.q.norm"][:-1]
    bad["l0.mlp.router.b"] = np.zeros(2)
    bad["extra"] = np.zeros(3)
    (tmp_path / "bad").mkdir()
    P.write_safetensors(tmp_path / "bad" / "model.safetensors", bad, "BF16")
    (tmp_path / "bad" / "config.json").write_text(json.dumps(U.CFG_B))
    arch, cfg, f = open_model_source(tmp_path / "bad")
    with pytest.raises(WeightsError) as e:
        plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    assert e.value.missing == ["l1.mix.right.out"] and e.value.unexpected == ["extra"]
    assert sorted(n for n, _, _ in e.value.wrong_shape) == ["l0.mlp.router.b", "l1.mix.left.q.norm"]


def test_scaled_frequencies_of_the_product_match_the_plain_ones():
    from transformer_amd.parts.position import scaled_frequencies
    for dims, base, sc in ((8, 1000.0, (8.0, 1.0, 4.0, 64)), (64, 5e5, (4.0, 1.0, 4.0, 2048)), (34, 20.0, (3.0, 1.0, 3.0, 32)),
                           (16, 1e4, None), (2, 7.0, (2.0, 0.5, 8.0, 4))):
        rot = U._rot(dims, base, sc)
        np.testing.assert_allclose(scaled_frequencies(dims, base, sc), P.rotation_frequencies(rot), rtol=1e-13)


# ---------------------------------------------------------------- the plain functions themselves
def test_plain_frequencies_keep_slow_and_blend():
    rot = U._rot(8, 1000.0, (8.0, 1.0, 4.0, 64))
    f = 1000.0 ** (-np.arange(4) / 4.0)
    got = P.rotation_frequencies(rot)
    wl = 2 * np.pi / f                                     # 6.3, 35, 199, 1117: below 16, between 16 and 64, above 64 twice
    assert wl[0] < 16 < wl[1] < 64 < wl[2]
    s = (64 / wl[1] - 1.0) / 3.0
    np.testing.assert_allclose(got, [f[0], (1 - s) * f[1] / 8 + s * f[1], f[2] / 8, f[3] / 8])
    np.testing.assert_allclose(P.rotation_frequencies(U._rot(8, 1000.0)), f)


def test_plain_rotation_pairs_halves_and_keeps_relative_angles():
    rng = np.random.default_rng(0)
    t = rng.standard_normal((5, 2, 12))
    rot = U._rot(8, 100.0)
    r = P.rotate_half(t, np.arange(5), rot)
    np.testing.assert_allclose(r[..., 8:], t[..., 8:])
    np.testing.assert_allclose(np.linalg.norm(r, axis=-1), np.linalg.norm(t, axis=-1))
    np.testing.assert_allclose(r[0], t[0])
    one = np.zeros((2, 1, 4))
    one[:, 0, 0] = 1.0                                     # coordinate 0 turns into coordinate 2, not 1
    np.testing.assert_allclose(P.rotate_half(one, [0, 1], U._rot(4, 10.0))[1, 0], [np.cos(1.0), 0, np.sin(1.0), 0])
    a = P.rotate_half(t, np.arange(5) + 9, rot)
    np.testing.assert_allclose(np.einsum("thd,shd->tsh", a, a), np.einsum("thd,shd->tsh", r, r), atol=1e-9)


def test_plain_linear_attention_equals_its_sum_form_and_carries_its_state():
    rng = np.random.default_rng(1)
    T, H, dk, dv = 9, 3, 4, 5
    q, k = rng.standard_normal((T, H, dk)), rng.standard_normal((T, H, dk))
    v = rng.standard_normal((T, H, dv))
    decay = [0.9, 1.0, 0.0]
    got, S = P.decayed_linear_attention(q, k, v, decay)
    np.testing.assert_allclose(got, P.decayed_linear_attention_sum(q, k, v, decay), atol=1e-12)
    a, S1 = P.decayed_linear_attention(q[:5], k[:5], v[:5], decay)
    b, S2 = P.decayed_linear_attention(q[5:], k[5:], v[5:], decay, S1)
    np.testing.assert_allclose(np.concatenate([a, b]), got, atol=1e-12)
    np.testing.assert_allclose(S2, S, atol=1e-12)
    # a decay of 0 sees the current token only
    np.testing.assert_allclose(got[:, 2], np.einsum("tk,tk->t", q[:, 2], k[:, 2])[:, None] * v[:, 2], atol=1e-12)


def test_plain_expert_limits_and_routing():
    w = {"gate": np.array([[1.0]]), "up": np.array([[1.0]]), "down": np.array([[1.0]])}
    for x, g, u in ((0.5, 0.5, 0.5), (3.0, 1.5, 1.5), (-3.0, -3.0, -1.5)):    # the gate is cut from above only
        want = g * P.sigmoid(1.702 * g) * (u + 1.0)
        np.testing.assert_allclose(P.expert(np.array([[x]]), w, "", 1.5), [[want]])
    z = np.array([[1.0, 3.0, 3.0, -1.0], [0.0, 0.0, 0.0, 0.0]])
    chosen, weight = P.route(z, 2)
    assert chosen.tolist() == [[1, 2], [0, 1]]             # the lowest index among equals
    np.testing.assert_allclose(weight, [[0.5, 0.5], [0.5, 0.5]])
    chosen, weight = P.route(z[:1], 3)
    e = np.exp([3.0, 3.0, 1.0])
    np.testing.assert_allclose(weight[0], e / e.sum())     # softmax over the chosen alone


def test_plain_model_is_causal_and_adds_both_sublayers_to_one_norm():
    cfg, seed = U.CONFIGS["B"]
    m = P.PlainLuduvik(config=cfg, weights=P.random_weights(cfg, seed))
    toks = U.tokens("B", 12, 0)
    a, b = m.forward(toks), m.forward(toks[:7])
    np.testing.assert_allclose(a[:7], b, atol=1e-10)
    layers = []
    m.forward(toks[:3], layers)
    w, eps = m.w, cfg["norm"]["eps"]
    x0 = w["embed"][toks[:3]]
    h = P.rms_norm(x0, w["l0.norm1"], eps)
    want = x0 + P.lightning_mixer(h, w, "l0.mix.", cfg["layers"][0]["mixer"], eps) + P.moe(h, w, "l0.mlp.", cfg["layers"][0]["mlp"])
    np.testing.assert_allclose(layers[0], want, atol=1e-12)


def test_bench_shapes_of_the_design_option_are_valid_models():
    import bench
    import transformer_amd as ta
    for size, (base, kinds, near) in bench.luduvik_shapes().items():
        for kind, layers in kinds.items():
            cfg = ta.LuduvikConfig.from_dict({**base, "layers": layers})
            spec = cfg.model_spec()
            assert len(spec.blocks) == len(layers) and spec.hidden == base["width"], (size, kind)
        for arch, cfg_dict in near.values():
            assert ta.get_architecture(arch).config_from_dict(cfg_dict).model_spec().hidden == base["width"]
