"""Kunitar without a GPU: configuration keys, the layout it spells out, where parameters are
found in a file, binding errors, and the plain implementation's own invariants."""
import copy
import json

import numpy as np
import pytest

import kunitar_util as U
import plain_kunitar as P


def _cfg(d):
    from transformer_amd.config.kunitar import KunitarConfig
    return KunitarConfig.from_dict(d)


def test_config_reads_every_key_and_writes_it_back():
    cfg = _cfg(U.CFG_A)
    assert (cfg.vocab, cfg.width, cfg.eps, cfg.embed_scale, cfg.side_dim) == (211, 72, 1e-5, 2.5, 12)
    a = cfg.layers[0]
    assert (a.type, a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.scale, a.rot_dims, a.rot_base,
            a.window, a.kv_from) == ("latent_attention", 3, 20, 8, 28, 40, 48, 0.2, 8, 1000.0, 33, None)
    assert (a.mlp, a.experts, a.top, a.ff, a.shared_ff) == ("moe", 5, 2, 24, 40)
    assert cfg.layers[2].kv_from == 0 and cfg.layers[2].mlp is None and cfg.layers[4].window is None
    assert (cfg.layers[1].decay_rank, cfg.layers[1].mlp, cfg.layers[1].ff) == (6, "dense", 100)
    assert cfg.layers[3].shared_ff is None and cfg.layers[3].top == 3
    assert _cfg(cfg.to_dict()) == cfg
    assert _cfg(U.CFG_B).side_dim is None and _cfg(U.CFG_D).layers[0].rot_dims == 4


def test_config_errors_name_the_key():
    from transformer_amd.config.spec import ConfigError
    for path, value in ((("layers", 0, "type"), "mamba"), (("layers", 0, "mlp", "kind"), "glu"),
                        (("layers", 2, "mixer", "kv_from"), 1), (("layers", 2, "mixer", "kv_from"), 2),
                        (("layers", 5, "mixer", "kv_from"), 2), (("layers", 2, "mixer", "kv_rank"), 40),
                        (("layers", 0, "mixer", "rot", "dims"), 10), (("layers", 0, "mlp", "router", "top"), 6),
                        (("layers", 0, "mixer", "mask", "size"), 0), (("norm",), None), (("token_side", "dim"), 0)):
        d = copy.deepcopy(U.CFG_A)
        at = d
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            _cfg(d)


def test_layout_schedule_windows_and_cache_needs():
    import torch
    from transformer_amd.cache.storage import KVNeed, StateNeed
    from transformer_amd.parts.base import build_part
    spec = _cfg(U.CFG_A).model_spec()
    assert [r.cache_of for r in spec.schedule] == [None, None, 0, None, None, 4]
    # rows are kept for the widest window among the layer that caches them and its readers
    assert [(b.mixer.window, b.mixer.cache_window, b.mixer.own_kv) for b in spec.blocks if b.mixer.kind == "latent_attention"] == \
        [(33, 70, True), (70, 70, False), (None, None, True), (20, None, False)]
    assert [b.ffn.kind if b.ffn is not None else None for b in spec.blocks] == \
        ["routed_mlp", "mlp", None, "routed_mlp", "routed_mlp", "mlp"]
    assert [b.side.offset for b in spec.blocks] == [0, 12, 24, 36, 48, 60]
    needs = [build_part(b, torch.float32, "cpu").cache_need() for b in spec.blocks]
    assert needs[0] == needs[2] == KVNeed(1, 56, 70, 0) and needs[4] == needs[5] == KVNeed(1, 32, None, 0)
    assert needs[1] == [StateNeed((72,)), StateNeed((3, 24, 24))]
    assert [p.kind for p in spec.after_embed.parts] == ["embed_scale", "token_side_table"]
    assert spec.after_embed.parts[1].width == 72 and spec.tie_embeddings is True
    assert _cfg(U.CFG_B).model_spec().after_embed is None


def test_every_parameter_has_a_file_tensor_and_back():
    from transformer_amd.config.registry import get_architecture
    from transformer_amd.engine.params import declared_params
    arch = get_architecture("Kunitar")
    for cfg_dict in (U.CFG_A, U.CFG_B, U.CFG_D):
        cfg = arch.config_from_dict(cfg_dict)
        params = declared_params(arch.model_spec(cfg))
        src = arch.weight_sources(cfg, "safetensors")
        assert set(src) == set(params)
        named = {}
        for pname, s in src.items():
            if not s.options:
                assert s.stand_in == "embed.weight"
                continue
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
    assert cfg.layers[0].decay_rank == 2 and cfg.layers[3].decay_rank == 5      # from the tensors' shapes
    plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    bad = dict(w)
    del bad["l0.mix.mu.g"]
    bad["l1.mix.dkv.norm"] = bad["l1.mix.dkv.norm"][:-1]
    bad["extra"] = np.zeros(3)
    (tmp_path / "bad").mkdir()
    P.write_safetensors(tmp_path / "bad" / "model.safetensors", bad, "BF16")
    (tmp_path / "bad" / "config.json").write_text(json.dumps(U.CFG_B))
    arch, cfg, f = open_model_source(tmp_path / "bad")
    with pytest.raises(WeightsError) as e:
        plan_binding(declared_params(arch.model_spec(cfg)), arch.weight_sources(cfg, f.format), f)
    assert e.value.missing == ["l0.mix.mu.g"] and e.value.unexpected == ["extra"]
    assert [n for n, _, _ in e.value.wrong_shape] == ["l1.mix.dkv.norm"]


# ---------------------------------------------------------------- the plain functions themselves
def test_plain_rotation_pairs_neighbours_and_keeps_relative_angles():
    rng = np.random.default_rng(0)
    t = rng.standard_normal((5, 2, 12))
    r = P.rotate_pairs(t, np.arange(5), 100.0, 8)
    np.testing.assert_allclose(r[..., 8:], t[..., 8:])
    np.testing.assert_allclose(np.linalg.norm(r, axis=-1), np.linalg.norm(t, axis=-1))
    np.testing.assert_allclose(r[0], t[0])
    one = np.zeros((2, 1, 4))
    one[:, 0, 0] = 1.0                                     # coordinate 0 turns into coordinate 1, not 2
    np.testing.assert_allclose(P.rotate_pairs(one, [0, 1], 10.0, 4)[1, 0], [np.cos(1.0), np.sin(1.0), 0, 0])
    a = P.rotate_pairs(t, np.arange(5) + 9, 100.0, 8)
    np.testing.assert_allclose(np.einsum("thd,shd->tsh", a, a), np.einsum("thd,shd->tsh", r, r), atol=1e-9)


def test_plain_recurrence_equals_its_sum_form():
    """o_t = sum_{s<t} (r_t . (k_s * prod_{s<j<t} w_j)) v_s + (r_t . (u * k_t)) v_t."""
    rng = np.random.default_rng(1)
    T, n = 8, 3
    r, k, v = (rng.standard_normal((T, 1, n)) for _ in range(3))
    w, u = rng.uniform(0.3, 0.9, (T, 1, n)), rng.standard_normal((1, n))
    got, S = P.wkv_recurrence(r, k, v, w, u)
    want = np.zeros((T, n))
    for t in range(T):
        for s in range(t):
            want[t] += (r[t, 0] @ (k[s, 0] * np.prod(w[s + 1:t, 0], axis=0))) * v[s, 0]
        want[t] += (r[t, 0] @ (u[0] * k[t, 0])) * v[t, 0]
    np.testing.assert_allclose(got[:, 0], want, atol=1e-12)
    a, S1 = P.wkv_recurrence(r[:5], k[:5], v[:5], w[:5], u)        # the state carries a cut
    b, S2 = P.wkv_recurrence(r[5:], k[5:], v[5:], w[5:], u, S1)
    np.testing.assert_allclose(np.concatenate([a, b]), got, atol=1e-12)
    np.testing.assert_allclose(S2, S, atol=1e-12)


def test_plain_routing_weights_inputs_and_picks_the_lowest_index_among_equals():
    h = np.array([[1.0, 0.0], [0.0, 2.0]])
    router = np.array([[1.0, 0.0], [1.0, 0.0], [0.0, 1.0]])
    chosen, weight = P.route(h, router, 2)
    assert chosen.tolist() == [[0, 1], [2, 0]]
    np.testing.assert_allclose(weight[1], [P.sigmoid(2.0), 0.5])
    w = {"router": np.array([[5.0, 0.0]]), "e0.up": np.array([[1.0, 0.0]]), "e0.down": np.array([[1.0], [0.0]])}
    out = P.moe(np.array([[2.0, 0.0]]), w, "", {"router": {"top": 1}})
    s = P.sigmoid(10.0)
    np.testing.assert_allclose(out, [[(2.0 * s) ** 2, 0.0]])       # the weight is squared with the input


def test_plain_window_and_activations():
    assert abs(P.gelu_erf(1.0) - 0.8413447460685429) < 1e-12 and abs(P.gelu_tanh(1.0) - 0.8411919906) < 1e-9
    assert P.relu_squared(-2.0) == 0.0 and P.relu_squared(3.0) == 9.0
    cfg, seed = U.CONFIGS["B"]
    m = P.PlainKunitar(config=cfg, weights=P.random_weights(cfg, seed))
    toks = U.tokens("B", 12, 0)
    a, b = m.forward(toks), m.forward(toks[:7])
    np.testing.assert_allclose(a[:7], b, atol=1e-10)               # causal


def test_bench_shapes_of_the_design_option_are_valid_models():
    import bench
    import transformer_amd as ta
    for size, (base, kinds, llama) in bench.kunitar_shapes().items():
        for kind, layers in kinds.items():
            cfg = ta.KunitarConfig.from_dict({**base, "layers": layers})
            spec = cfg.model_spec()
            assert len(spec.blocks) == len(layers) and spec.hidden == base["width"], (size, kind)
        lc = ta.LlamaConfig.from_dict({**llama, "num_hidden_layers": 2})
        assert lc.hidden == base["width"]
