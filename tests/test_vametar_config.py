"""Vametar without a GPU: configuration keys, the layout it spells out, where parameters are
found in a file, binding errors, and the plain implementation's own invariants."""
import copy
import json

import numpy as np
import pytest

import plain_vametar as P
import vametar_util as U


def _cfg(d):
    from transformer_amd.config.vametar import VametarConfig
    return VametarConfig.from_dict(d)


def test_config_reads_every_key_and_writes_it_back():
    cfg = _cfg(U.CFG_A)
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.residual_mult, cfg.logit_scale) == (331, 96, 1e-5, 0.5, 1.5)
    assert (cfg.buckets, cfg.mul_prev, cfg.mul_cur) == (97, 13, 5)
    a = cfg.layers[0]
    assert (a.type, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base, a.v_mix, a.ff) == \
        ("attention", 6, 3, 40, 24, 16, 1000.0, True, 136)
    assert cfg.layers[4].kv_heads == 4 and cfg.layers[4].rot_dims == 0 and not cfg.layers[4].v_mix
    assert cfg.layers[1].rank == 5 and cfg.layers[2].conv == 4 and cfg.layers[1].ff is None
    assert _cfg(cfg.to_dict()) == cfg


def test_config_errors_name_the_key():
    from transformer_amd.config.spec import ConfigError
    for path, value in ((("layers", 0, "type"), "mamba"), (("layers", 0, "mlp", "kind"), "moe"),
                        (("layers", 2, "mixer", "blocks"), 5), (("layers", 0, "mixer", "kv_heads"), 4),
                        (("norm",), None), (("embedding", "bigram", "buckets"), 0)):
        d = copy.deepcopy(U.CFG_A)
        at = d
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            _cfg(d)


def test_layout_roles_of_value_mixing_and_cache_needs():
    import torch
    from transformer_amd.cache.storage import KVNeed, StateNeed
    from transformer_amd.parts.base import build_part
    spec = _cfg(U.CFG_A).model_spec()
    roles = [getattr(b.mixer, "value_mix", "-") for b in spec.blocks]
    assert roles == ["source", "-", "-", "mix", None, "mix", "-"]
    assert [b.ffn is not None for b in spec.blocks] == [True, False, True, False, False, True, True]
    needs = [build_part(b, torch.float32, "cpu").cache_need() for b in spec.blocks]
    assert needs[0] == [StateNeed((96,)), KVNeed(3, 40, None, 24)]
    assert needs[1] == [StateNeed((96,)), StateNeed((3, 20, 28))]
    assert needs[2] == [StateNeed((96,)), StateNeed((144,)), StateNeed((3, 144))]
    assert spec.after_embed.buckets == 97 and spec.on_logits.scale == 1.5
    assert _cfg(U.CFG_B).model_spec().on_logits is None


def test_every_parameter_has_a_file_tensor_and_back():
    from transformer_amd.config.registry import get_architecture
    from transformer_amd.engine.params import declared_params
    arch = get_architecture("Vametar")
    for cfg_dict in (U.CFG_A, U.CFG_B):
        cfg = arch.config_from_dict(cfg_dict)
        params = declared_params(arch.model_spec(cfg))
        src = arch.weight_sources(cfg, "safetensors")
        assert set(src) == set(params)
        named = {}
        for pname, s in src.items():
            rows = sum(p.shape[0] for p in s.options[0]) if params[pname].shape else 0
            assert not params[pname].shape or rows == params[pname].shape[0], pname
            named.update({p.name: p.shape for p in s.options[0]})
        assert named == {n: tuple(s) for n, s in P.tensor_shapes(cfg_dict).items()}


def test_loader_reports_missing_and_misshaped_tensors(tmp_path):
    from transformer_amd.api import open_model_source
    from transformer_amd.engine.params import declared_params
    from transformer_amd.weights.loader import WeightsError, plan_binding
    w = P.make_model_folder(tmp_path / "ok", U.CFG_B, 1)
    arch, cfg, f = open_model_source(tmp_path / "ok")
    assert cfg.layers[1].rank == 2
    plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    bad = dict(w)
    del bad["l0.shift"]
    bad["l2.mix.q.norm"] = bad["l2.mix.q.norm"][:-1]
    bad["extra"] = np.zeros(3)
    (tmp_path / "bad").mkdir()
    P.write_safetensors(tmp_path / "bad" / "model.safetensors", bad, "BF16")
    (tmp_path / "bad" / "config.json").write_text(json.dumps(U.CFG_B))
    arch, cfg, f = open_model_source(tmp_path / "bad")
    with pytest.raises(WeightsError) as e:
        plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    assert e.value.missing == ["l0.shift"] and e.value.unexpected == ["extra"]
    assert [n for n, _, _ in e.value.wrong_shape] == ["l2.mix.q.norm"]


# ---------------------------------------------------------------- the plain functions themselves
def test_plain_token_shift_and_pair_rows():
    h = np.arange(12.0).reshape(4, 3)
    np.testing.assert_allclose(P.token_shift(h, np.array([0.0, 1.0, 0.5])),
                               [[0, 0, 1], [3, 1, 3.5], [6, 4, 6.5], [9, 7, 9.5]])
    assert list(P.bigram_rows([3, 4, 4], 10, 7, 2)) == [10, (21 + 8) % 10, (28 + 8) % 10]


def test_plain_rotation_keeps_lengths_and_relative_angles():
    rng = np.random.default_rng(0)
    t = rng.standard_normal((5, 2, 12))
    r = P.rotate_partial(t, np.arange(5), 100.0, 8)
    np.testing.assert_allclose(r[..., 8:], t[..., 8:])
    np.testing.assert_allclose(np.linalg.norm(r, axis=-1), np.linalg.norm(t, axis=-1))
    np.testing.assert_allclose(r[0], t[0])
    a = P.rotate_partial(t, np.arange(5) + 9, 100.0, 8)
    np.testing.assert_allclose(np.einsum("thd,shd->tsh", a, a), np.einsum("thd,shd->tsh", r, r), atol=1e-9)


def test_plain_linear_attention_equals_its_sum_form():
    """o_t = sum_{s<=t} (q_t . (k_s * prod_{s<r<=t} alpha_r)) v_s."""
    rng = np.random.default_rng(1)
    T, d, dk, dv, r = 9, 6, 4, 3, 2
    m = {"heads": 1, "dim": dk, "vdim": dv, "tau": 2.0}
    w = {"p.q": rng.standard_normal((dk, d)), "p.k": rng.standard_normal((dk, d)), "p.v": rng.standard_normal((dv, d)),
         "p.g": rng.standard_normal((dv, d)), "p.o": np.eye(dv), "p.norm": np.ones(dv), "p.a1": rng.standard_normal((r, d)),
         "p.a2": rng.standard_normal((dk, r)), "p.a2.b": rng.standard_normal(dk)}
    h = rng.standard_normal((T, d))
    got = P.gla_mixer(h, w, "p.", m, 1e-6)
    q, k, v = (h @ w["p.q"].T) * dk ** -0.5, h @ w["p.k"].T, h @ w["p.v"].T
    alpha = P.sigmoid((h @ w["p.a1"].T) @ w["p.a2"].T + w["p.a2.b"]) ** 0.5
    o = np.zeros((T, dv))
    for t in range(T):
        for s in range(t + 1):
            o[t] += (q[t] @ (k[s] * np.prod(alpha[s + 1:t + 1], axis=0))) * v[s]
    np.testing.assert_allclose(got, P.unit_rms(o, 1e-6) * P.silu(h @ w["p.g"].T), atol=1e-10)


def test_plain_recurrence_bounds_and_convolution():
    x = np.arange(8.0).reshape(4, 2)
    taps = np.array([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]])
    np.testing.assert_allclose(P.causal_conv(x, taps, np.array([0.5, 0.0])),
                               [[0.5, 1], [200.5, 3], [420.5, 5], [642.5, 7]])
    assert abs(P.gelu_tanh(1.0) - 0.8411919906) < 1e-9 and P.gelu_tanh(0.0) == 0.0


def test_plain_model_is_causal():
    cfg, seed = U.CONFIGS["B"]
    m = P.PlainVametar(config=cfg, weights=P.random_weights(cfg, seed))
    toks = U.tokens("B", 12, 0)
    a, b = m.forward(toks), m.forward(toks[:7])
    np.testing.assert_allclose(a[:7], b, atol=1e-10)


def test_bench_shapes_of_the_design_option_are_valid_models():
    """``bench.py --design vametar`` builds these: every layer kind alone and the Llama layer of
    the same width, heads and feed-forward."""
    import bench
    import transformer_amd as ta
    for size, (base, kinds, llama) in bench.vametar_shapes().items():
        for kind, layer in kinds.items():
            cfg = ta.VametarConfig.from_dict({**base, "layers": [layer] * 2})
            spec = cfg.model_spec()
            assert len(spec.blocks) == 2 and spec.hidden == base["width"], (size, kind)
        lc = ta.LlamaConfig.from_dict({**llama, "num_hidden_layers": 2})
        att = kinds["attention"]["mixer"]
        assert (lc.hidden, lc.num_heads, lc.num_kv_heads, lc.head_dim) == \
            (base["width"], att["heads"], att["kv_heads"], att["dim"])
        assert lc.intermediate == kinds["attention"]["mlp"]["ff"]
