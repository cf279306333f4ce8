"""The Zogurax design without a GPU: the configuration reader, the model's description (tensors, runs,
cache units), the plain implementation's mechanisms against numbers worked by hand or against
themselves continued from a carried state, and random models written and read back."""
import copy
import importlib
import json
import os

import numpy as np
import pytest

import plain_zogurax as pz
import zogurax_configs as zc

L = importlib.import_module("daisi-llogos_amd")
registry = importlib.import_module("daisi-llogos_amd.config.registry")
model_mod = importlib.import_module("daisi-llogos_amd.models.model")
config_mod = importlib.import_module("daisi-llogos_amd.config.model_config")


def _model(cfg):
    arch = registry.architecture_of(cfg)
    return arch.read_config(cfg), model_mod.Model(arch.model_spec(arch.read_config(cfg)))


def test_the_reader_takes_every_size_and_constant_from_the_file():
    typed, _ = _model(zc.ZOG_A)
    assert (typed.vocab, typed.width, typed.norm_eps) == (211, 96, 1e-5)
    assert [l.type for l in typed.layers] == ["attention_2", "attention", "attention_2", "attention"]
    m = typed.layers[1].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.softcap, m.temp_coef, m.temp_every, m.conv) == (3, 3, 16, 40, 0.4, 2.0, 0.4, 7, 3)
    assert typed.layers[0].mixer.conv == 0 and typed.layers[2].mlp is None
    f = typed.layers[1].mlp
    assert (f.experts, f.top, f.ff, f.shared_ff) == (4, 3, 24, 56)
    assert (typed.loop.start, typed.loop.stop, typed.loop.times) == (1, 3, 3)
    assert _model(zc.ZOG_B)[0].loop is None


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "attention_3", "attention_3"), (("layers", 1, "mixer", "conv"), -1, "conv"),
    (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 0, "mlp", "kind"), "dense", "dense"),
    (("layers", 0, "mlp", "router", "top"), 9, "top"), (("loop", "stop"), 7, "loop"), (("loop", "times"), 0, "loop"),
    (("layers", 0, "mixer", "q_temp", "every"), 0, "every"), (("norm",), None, "norm"), (("width",), "wide", "width")])
def test_a_wrong_or_missing_key_is_named(path, value, word):
    cfg = copy.deepcopy(zc.ZOG_A)
    at = cfg
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(config_mod.ConfigError) as e:
        _model(cfg)
    assert word in str(e.value)


def test_the_description_runs_looped_layers_again_with_a_cache_of_their_own():
    _, model = _model(zc.ZOG_A)
    assert [e.layer for e in model.schedule] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [e.enter for e in model.schedule] == [None, (0, 0), None, (0, 1), None, (0, 2), None, None]
    assert [(l, t) for l, t in pz.layer_runs(zc.ZOG_A)] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    needs = model.cache_needs()
    assert len(needs) == 8 and model.cache_reads() == [None] * 8
    kv, st = needs[1]
    assert (kv.n_kv_heads, kv.head_dim, kv.value_dim) == (3, 16, 48)          # values of 40 in rows of 48
    assert st.shape == (2, 3 * 16 + 3 * 16 + 3 * 40)                          # the convolution's last two projected rows
    assert needs[0][1] is None and needs[3] == needs[1] and needs[5] == needs[1]
    names = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert names["loop.in"] == (96, 192) and names["loop.step"] == (3, 96) and names["head"] == (211, 96)
    assert names["l0.mix.q.b"] == (128,) and names["l0.mix.o.b"] == (96,) and "l0.mix.g" not in names
    assert names["l1.mix.g"] == (3, 96) and names["l1.mix.q.norm"] == (48,) and names["l1.mix.v.conv"] == (120, 3)
    assert names["l1.mlp.table"] == (211, 3) and names["l1.mlp.e3.down"] == (96, 24) and names["l1.mlp.shared.sg"] == (1, 96)
    assert not any(n.startswith("l2.mlp") for n in names)
    _, plain_model = _model(zc.ZOG_B)
    assert [e.layer for e in plain_model.schedule] == [0, 1, 2] and not plain_model.stream_parts


def test_a_random_model_is_written_and_read_back(tmp_path):
    path = L.write_random_model(str(tmp_path / "m"), zc.ZOG_D, seed=3)
    cfg, w = pz.load_folder(path)
    assert cfg == zc.ZOG_D
    table = w["l1.mlp.table"]
    assert table.dtype == np.int32 and table.shape == (67, 4) and table.min() >= 0 and table.max() < 7
    assert all(len(set(row)) == 4 for row in table.tolist())                  # a row's experts differ
    assert len({tuple(r) for r in table.tolist()}) > 3
    logits = pz.forward(cfg, w, [1, 5, 66, 0, 5])
    assert logits.shape == (5, 67) and np.isfinite(logits).all()
    again = L.write_random_model(str(tmp_path / "n"), zc.ZOG_D, seed=3)
    assert all(np.array_equal(w[k], v) for k, v in pz.load_folder(again)[1].items())


def test_the_position_vector_by_hand():
    v = pz.position_vector([0, 3], 6)
    assert np.allclose(v[0], [0, 1, 0, 1, 0, 1])
    f = [1.0, 10000.0 ** (-2 / 6), 10000.0 ** (-4 / 6)]
    assert np.allclose(v[1], [np.sin(3 * f[0]), np.cos(3 * f[0]), np.sin(3 * f[1]), np.cos(3 * f[1]), np.sin(3 * f[2]), np.cos(3 * f[2])])
    assert pz.position_vector([2], 5).shape == (1, 5)                         # an odd width ends on a sine


def test_the_layer_norm_and_the_query_factor_by_hand():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    out = pz.layer_norm(x, np.array([1.0, 2.0, 1.0, 0.5]), 0.5)
    assert np.allclose(out, (x - 3.0) / np.sqrt(3.5 + 0.5) * [1.0, 2.0, 1.0, 0.5])
    t = pz.query_temperature([0, 1, 2, 5, 6, 20], 0.5, 3)
    assert np.allclose(t, 1 + 0.5 * np.log(np.array([0, 0, 1, 2, 2, 7]) + 1.0))


def test_the_unit_in_the_denominator_and_the_bend_by_hand():
    q = np.array([[[2.0]], [[1.0]]])                                          # two positions, one head of one dimension
    k = np.array([[[1.0]], [[3.0]]])
    v = np.array([[[10.0]], [[20.0]]])
    out = pz.causal_attention(q, k, v, 0.5, None, unit_sink=True)
    e0 = np.exp(1.0)
    assert np.isclose(out[0, 0, 0], 10 * e0 / (1 + e0))
    a, b = np.exp(0.5), np.exp(1.5)
    assert np.isclose(out[1, 0, 0], (10 * a + 20 * b) / (1 + a + b))
    bent = pz.causal_attention(q, k, v, 0.5, 1.0, unit_sink=False)
    a, b = np.exp(np.tanh(0.5)), np.exp(np.tanh(1.5))
    assert np.isclose(bent[1, 0, 0], (10 * a + 20 * b) / (a + b)) and np.isclose(bent[0, 0, 0], 10.0)


def test_the_convolution_continues_from_the_rows_before():
    rng = np.random.default_rng(0)
    u, w = rng.standard_normal((9, 4)), rng.standard_normal((4, 3))
    whole = pz.time_convolution(u, w)
    assert np.allclose(whole[0], w[:, 2] * u[0]) and np.allclose(whole[1], w[:, 1] * u[0] + w[:, 2] * u[1])
    assert np.allclose(pz.time_convolution(u[5:], w, before=u[3:5]), whole[5:])
    assert np.allclose(pz.time_convolution(u, w[:, -1:]), u * w[:, -1])       # one tap: a factor a channel


def test_the_mixture_takes_the_tables_experts_with_equal_weights():
    rng = np.random.default_rng(1)
    h = rng.standard_normal((3, 4))
    ups, downs = [rng.standard_normal((5, 4)) for _ in range(3)], [rng.standard_normal((4, 5)) for _ in range(3)]
    table = np.array([[0, 2], [1, 0], [2, 1]])
    out = pz.table_mixture(h, [2, 0, 2], table, ups, downs)
    want0 = (pz.expert(h[:1], ups[2], downs[2]) + pz.expert(h[:1], ups[1], downs[1]))[0] / 2
    assert np.allclose(out[0], want0) and np.allclose(out[2], (pz.expert(h[2:], ups[2], downs[2]) + pz.expert(h[2:], ups[1], downs[1]))[0] / 2)
    assert np.allclose(pz.squared_relu(np.array([-1.0, 0.5])), [0.0, 0.25])
    gate = rng.standard_normal((1, 4))
    assert np.allclose(pz.gated_shared_expert(h, ups[0], downs[0], gate), pz.expert(h, ups[0], downs[0]) / (1 + np.exp(-(h @ gate.T))))


def test_the_loop_entry_reads_the_stream_first_and_the_embedding_second():
    x, x0 = np.array([[1.0, 2.0]]), np.array([[10.0, 20.0]])
    w_in = np.array([[1.0, 0.0, 0.0, 0.0], [0.0, 0.0, 0.0, 1.0]])
    assert np.allclose(pz.loop_entry(x, x0, w_in, np.array([0.5, -0.5])), [[1.5, 19.5]])
